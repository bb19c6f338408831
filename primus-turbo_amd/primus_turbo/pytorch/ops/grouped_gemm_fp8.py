"""``grouped_gemm_fp8``: MoE grouped linear layer in FP8 with autograd
(reference: primus_turbo/pytorch/ops/grouped_gemm_fp8.py:99-265,853-960).

TENSORWISE / ROWWISE (reference :265-603): the packed rows of all groups are quantized as one
tensor (one scale, or one per token row / weight row); the vector scales are applied in the GEMM
epilogue.

BLOCKWISE (128): one fused pass over the bf16 activation yields the row quantization (forward /
dgrad operand) and the segment-padded column quantization (wgrad operand); the weight is
quantized in 128 x 128 tiles that serve forward and backward unchanged.

MX_BLOCKWISE (MXFP8, reference :604-840): activations and gradients go through the grouped MX
quantizer (rows padded to 32 per group, transposed columns to 128), weights through the dense MX
quantizer with 32 x 32 blocks in both directions; forward and dgrad are row-group NT products
whose output is packed by the tight offsets, wgrad is a variable-K NT product over the padded
column-direction operands. NT only (``trans_b=True``).
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from primus_turbo.pytorch.core.backend import BackendType
from primus_turbo.pytorch.core.low_precision import (
    Float8QuantConfig,
    ScalingGranularity,
    ScalingRecipe,
)
from primus_turbo.pytorch.core.quantized_tensor import (
    QuantizedTensor,
    QuantizedTensorPair,
    check_quantized_tensor,
)
from primus_turbo.pytorch.kernels.grouped_gemm.grouped_gemm_fp8_impl import (
    grouped_gemm_fp8_impl,
    grouped_gemm_fp8_variable_k_accum_impl,
    grouped_gemm_fp8_variable_k_impl,
)
from primus_turbo.pytorch.kernels.grouped_gemm.grouped_gemm_utils import group_offs_from_lens
from primus_turbo.pytorch.kernels.quantization.quantization_impl import (
    glu_grouped_quantize_mx_impl,
    glu_quant_fp8_blockwise_segment_m_row_col_impl,
    grouped_quantize_mxfp8_impl,
    quant_fp8_blockwise_for_weight_dual_impl,
    quant_fp8_blockwise_for_weight_impl,
    quant_fp8_blockwise_segment_m_row_col_impl,
    quant_fp8_blockwise_segment_m_row_col_t_impl,
    quantize_mxfp8_impl,
)
from primus_turbo.pytorch.ops.quantization import dequantize_fp8, quantize_fp8
from primus_turbo.pytorch.ops.utils import (
    _ensure_contiguous_grad_out,
    _get_dummy_wgrad,
    _get_fp8_dtype,
    _setup_fused_grad_accum,
)

__all__ = ["grouped_gemm_fp8", "glu_grouped_gemm_fp8"]

_NATIVE = BackendType.TRITON.value  # placeholder id: a single backend exists here


def _grouped_gemm_fp8_variable_k_impl_wrapper(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b,
                                              trans_c, out_dtype, granularity, num_cu, default_backend,
                                              inplace_add_to_out=False, out=None):
    """Variable-K wgrad GEMM; with ``inplace_add_to_out`` the product is added into ``out``
    (fp32 ``main_grad``) and a placeholder in the weight's dtype is returned for autograd."""
    if not inplace_add_to_out:
        return grouped_gemm_fp8_variable_k_impl(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b,
                                                trans_c, out_dtype, granularity, num_cu, default_backend)
    assert out is not None, "out should not be None when inplace_add_to_out is True"
    grouped_gemm_fp8_variable_k_accum_impl(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b,
                                           trans_c, out.dtype, granularity, num_cu, default_backend, out)
    return _get_dummy_wgrad(out.shape, out_dtype)


def _block_forward_product(a_fp8_row, a_scale_row, b, group_lens, group_offs, trans_b, out_dtype, config, num_cu, need_bwd):
    """Quantize the BLOCKWISE weight (2-D blocks; with the transposed copy for the backward product
    when it is needed and possible) and multiply -> ``(out, (weight codes, scales) for dgrad,
    whether those are K-contiguous for dgrad already)``."""
    bs = config.block_size
    b_dtype = _get_fp8_dtype(config.format, True)
    b_recipe = ScalingRecipe(use_2d_block=True)
    b_fp8_t = None
    if isinstance(b, QuantizedTensor):
        check_quantized_tensor(b, config, scaling_recipe=b_recipe)
        b_fp8, b_scale = b.qdata, b.scale_inv
    elif (need_bwd or not trans_b) and b.size(-2) % 16 == 0:
        b_fp8, b_fp8_t, b_scale = quant_fp8_blockwise_for_weight_dual_impl(b, b_dtype, block_size=bs)
    else:
        b_fp8, b_scale = quant_fp8_blockwise_for_weight_impl(b, b_dtype, block_size=bs)

    # fwd reduces over b's last axis when trans_b, else over its middle axis
    fwd_b, dgrad_b = (b_fp8, b_fp8_t) if trans_b else (b_fp8_t, b_fp8)
    b_scale_t = b_scale.transpose(-2, -1).contiguous() if b_fp8_t is not None else None
    fwd_s, dgrad_s = (b_scale, b_scale_t) if trans_b else (b_scale_t, b_scale)
    if fwd_b is not None:
        out = grouped_gemm_fp8_impl(a_fp8_row, fwd_b, a_scale_row, fwd_s, group_lens, group_offs, False, True,
                                    out_dtype, config.granularity.value, num_cu, _NATIVE)
    else:
        out = grouped_gemm_fp8_impl(a_fp8_row, b_fp8, a_scale_row, b_scale, group_lens, group_offs, False, trans_b,
                                    out_dtype, config.granularity.value, num_cu, _NATIVE)
    if dgrad_b is not None:
        return out, (dgrad_b, dgrad_s), True
    return out, (b_fp8, b_scale), False


def _block_backward_products(grad_out, a_fp8_col_t, a_scale_col, b_fp8, b_scale, group_lens, group_offs, trans_b, config,
                             dgrad_dtype, wgrad_dtype, num_cu, b_ready, fuse_bgrad_accum, main_grad):
    """dgrad and variable-K wgrad of the BLOCKWISE grouped layer -> ``(grad_a, grad_b)``; the
    activation gradient comes out in ``dgrad_dtype``, the weight gradient in ``wgrad_dtype``."""
    g_dtype = _get_fp8_dtype(config.format, False)
    gran = config.granularity.value
    g_row, g_col_t, g_scale_row, g_scale_col, var_k_lens, var_k_offs = quant_fp8_blockwise_segment_m_row_col_t_impl(
        grad_out, g_dtype, config.block_size, group_lens, group_offs)
    # grad_a = grad_out @ b^T: the saved weight copy is contiguous along the reduction already,
    # or (caller-quantized weight) the forward operand read the other way round
    grad_a = grouped_gemm_fp8_impl(g_row, b_fp8, g_scale_row, b_scale, group_lens, group_offs, False,
                                   True if b_ready else not trans_b, dgrad_dtype, gran, num_cu, _NATIVE)
    # grad_b[g] = a_g^T @ grad_out_g over the padded token ranges, both operands K-major
    grad_b = _grouped_gemm_fp8_variable_k_impl_wrapper(
        a_fp8_col_t, g_col_t, a_scale_col, g_scale_col, var_k_lens, var_k_offs, False, True, trans_b, wgrad_dtype, gran,
        num_cu, _NATIVE, inplace_add_to_out=fuse_bgrad_accum, out=main_grad,
    )
    return grad_a, grad_b


class FP8GroupedGemmBlockFunc(torch.autograd.Function):
    """BLOCKWISE grouped GEMM autograd."""

    @staticmethod
    def forward(ctx, a, b, a_t, b_t, group_lens, group_offs, trans_b, out_dtype, config, num_cu,
                fuse_bgrad_accum_pattern=None):
        fuse_bgrad_accum, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        assert config.granularity == ScalingGranularity.BLOCKWISE
        assert config.block_size in [128], "Only block_size 128 is supported currently."
        if isinstance(a, QuantizedTensor):
            raise NotImplementedError("FP8GroupedGemmBlockFunc does not support a pre-quantized activation `a`")
        assert a.ndim == 2, "Input tensor must be 2-dimensional."
        assert b.ndim == 3, "Weight tensor must be 3-dimensional."
        assert group_lens.size(0) == b.size(0), "group_lens size must match b size(0)."
        assert out_dtype in [torch.float16, torch.bfloat16]
        a_dtype = _get_fp8_dtype(config.format, True)
        b_dtype = _get_fp8_dtype(config.format, True)

        need_bwd = any(ctx.needs_input_grad[:2])
        bs = config.block_size
        # Backward reduces over the tokens (wgrad) and over the other weight axis (dgrad): the
        # quantizers emit those operands K-contiguous from the same read, so that no GEMM has to
        # transpose anything. (A caller-quantized weight has no such copy: the GEMM transposes it.)
        if need_bwd:
            a_fp8_row, a_fp8_col_t, a_scale_row, a_scale_col, _, _ = quant_fp8_blockwise_segment_m_row_col_t_impl(
                a.contiguous(), a_dtype, bs, group_lens, group_offs)
        else:
            a_fp8_row, _, a_scale_row, _, _, _ = quant_fp8_blockwise_segment_m_row_col_impl(
                a.contiguous(), a_dtype, bs, group_lens, group_offs)
            a_fp8_col_t = a_scale_col = None
        out, saved_b, b_ready = _block_forward_product(a_fp8_row, a_scale_row, b, group_lens, group_offs, trans_b, out_dtype,
                                                       config, num_cu, need_bwd)
        if need_bwd:
            ctx.save_for_backward(a_fp8_col_t, a_scale_col, saved_b[0], saved_b[1], group_lens, group_offs)
        ctx.meta = (trans_b, config, out_dtype, num_cu, fuse_bgrad_accum, main_grad, b_ready)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = _ensure_contiguous_grad_out(grad_out)
        a_fp8_col_t, a_scale_col, b_fp8, b_scale, group_lens, group_offs = ctx.saved_tensors
        trans_b, config, out_dtype, num_cu, fuse_bgrad_accum, main_grad, b_ready = ctx.meta
        grad_a, grad_b = _block_backward_products(grad_out, a_fp8_col_t, a_scale_col, b_fp8, b_scale, group_lens, group_offs,
                                                  trans_b, config, out_dtype, out_dtype, num_cu, b_ready, fuse_bgrad_accum,
                                                  main_grad)
        return grad_a, grad_b, None, None, None, None, None, None, None, None, None


class FP8GluGroupedGemmBlockFunc(torch.autograd.Function):
    """Gated activation -> BLOCKWISE grouped GEMM (fc2 of an MoE expert MLP) with the activation
    fused into the quantizer of the GEMM's activation operand: the bf16 activation is neither
    written nor re-read, forward or backward (wgrad uses the column codes saved by the fused
    quantizer, the activation backward needs fc1's output only)."""

    @staticmethod
    def forward(ctx, x, probs, row_mask, act_type, b, group_lens, group_offs, trans_b, out_dtype, config, num_cu,
                fuse_bgrad_accum_pattern=None):
        fuse_bgrad_accum, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        assert config.granularity == ScalingGranularity.BLOCKWISE and config.block_size in [128]
        assert x.ndim == 2 and x.size(1) % 2 == 0, "x must be [tokens, 2 * hidden]"
        assert b.ndim == 3 and group_lens.size(0) == b.size(0)
        assert probs.dtype == torch.float32 and probs.numel() == x.size(0), "probs must be float32, one per token"
        assert out_dtype in [torch.float16, torch.bfloat16]
        need_bwd = any(ctx.needs_input_grad[i] for i in (0, 1, 4))
        x2, p1 = x.contiguous(), probs.reshape(-1).contiguous()
        a_fp8_row, a_col, a_scale_row, a_scale_col, _, _ = glu_quant_fp8_blockwise_segment_m_row_col_impl(
            x2, p1, row_mask, act_type, _get_fp8_dtype(config.format, True), config.block_size, group_lens, group_offs,
            need_bwd)
        out, saved_b, b_ready = _block_forward_product(a_fp8_row, a_scale_row, b, group_lens, group_offs, trans_b, out_dtype,
                                                       config, num_cu, need_bwd)
        if need_bwd:
            ctx.save_for_backward(x2, p1, row_mask, a_col, a_scale_col, saved_b[0], saved_b[1], group_lens, group_offs)
        ctx.meta = (trans_b, config, out_dtype, num_cu, fuse_bgrad_accum, main_grad, b_ready, act_type, probs.shape)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        from primus_turbo.pytorch.kernels.activation.glu_impl import ACT_GELU, ACT_SILU, glu_bwd_with_probs

        grad_out = _ensure_contiguous_grad_out(grad_out)
        x2, p1, row_mask, a_col_t, a_scale_col, b_fp8, b_scale, group_lens, group_offs = ctx.saved_tensors
        trans_b, config, out_dtype, num_cu, fuse_bgrad_accum, main_grad, b_ready, act_type, probs_shape = ctx.meta
        grad_act, grad_b = _block_backward_products(grad_out, a_col_t, a_scale_col, b_fp8, b_scale, group_lens, group_offs,
                                                    trans_b, config, x2.dtype, out_dtype, num_cu, b_ready, fuse_bgrad_accum,
                                                    main_grad)
        grad_x, grad_probs = glu_bwd_with_probs(grad_act, x2, p1, row_mask, ACT_SILU if act_type == "silu" else ACT_GELU)
        return grad_x, grad_probs.view(probs_shape), None, None, grad_b, None, None, None, None, None, None, None


def _quantize_plain(x, config, fwd: bool, axis: int):
    """-> ``(codes, scale_inv, original dtype)``. TENSORWISE / ROWWISE quantization treats the
    packed rows of all groups as one tensor (reference: core/quantized_tensor.py:309-325). Plain
    tensors rather than wrappers, so that ``torch.compile`` traces the functions below into one graph."""
    if isinstance(x, QuantizedTensor):
        check_quantized_tensor(x, config, axis=None if config.granularity == ScalingGranularity.TENSORWISE else axis)
        return x.qdata, x.scale_inv, x.dtype
    q, s = quantize_fp8(x.contiguous(), _get_fp8_dtype(config.format, fwd), config.granularity, axis=axis % x.ndim,
                        block_size=config.block_size)
    return q, s, x.dtype


class FP8GroupedGemmRowFunc(torch.autograd.Function):
    """ROWWISE grouped GEMM autograd (reference :265-447): activations scaled per token row, weights
    per output row of every expert; the operands of the backward GEMMs are re-quantized along
    their other axis from the de-quantized forward operands."""

    @staticmethod
    def forward(ctx, a, b, a_t, b_t, group_lens, group_offs, trans_b, out_dtype, config, num_cu,
                fuse_bgrad_accum_pattern=None):
        fuse_bgrad_accum, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        assert config.granularity == ScalingGranularity.ROWWISE
        b_row_axis, b_col_axis = (-1, -2) if trans_b else (-2, -1)
        qa, qa_s, a_hp = _quantize_plain(a, config, True, -1)
        qb, qb_s, b_hp = _quantize_plain(b, config, True, b_row_axis)
        gran = config.granularity.value
        out = grouped_gemm_fp8_impl(qa, qb, qa_s, qb_s, group_lens, group_offs, False, trans_b, out_dtype, gran, num_cu,
                                    _NATIVE)
        if any(ctx.needs_input_grad[:2]):
            def other_axis(q, q_s, hp_dtype, from_axis, given, axis):
                if given is not None:
                    assert isinstance(given, QuantizedTensor)
                    return given.qdata, given.scale_inv
                hp = dequantize_fp8(q, hp_dtype, config.granularity, axis=from_axis % q.ndim, scale_inv=q_s,
                                    block_size=config.block_size)
                return quantize_fp8(hp, q.dtype, config.granularity, axis=axis % q.ndim, block_size=config.block_size)

            a_col, a_col_s = other_axis(qa, qa_s, a_hp, -1, a_t, -2)
            b_col, b_col_s = other_axis(qb, qb_s, b_hp, b_row_axis, b_t, b_col_axis)
            ctx.save_for_backward(a_col, b_col, a_col_s, b_col_s, group_lens, group_offs)
        ctx.meta = (trans_b, config, out_dtype, num_cu, fuse_bgrad_accum, main_grad)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = _ensure_contiguous_grad_out(grad_out)
        a_col, b_col, a_col_s, b_col_s, group_lens, group_offs = ctx.saved_tensors
        trans_b, config, out_dtype, num_cu, fuse_bgrad_accum, main_grad = ctx.meta
        gran = config.granularity.value
        g_row, g_row_s, _ = _quantize_plain(grad_out, config, False, -1)
        grad_a = grouped_gemm_fp8_impl(g_row, b_col, g_row_s, b_col_s, group_lens, group_offs, False, not trans_b,
                                       out_dtype, gran, num_cu, _NATIVE)
        g_col, g_col_s, _ = _quantize_plain(grad_out, config, False, -2)
        grad_b = _grouped_gemm_fp8_variable_k_impl_wrapper(
            a_col, g_col, a_col_s, g_col_s, group_lens, group_offs, True, False, trans_b, out_dtype, gran,
            num_cu, _NATIVE, inplace_add_to_out=fuse_bgrad_accum, out=main_grad,
        )
        return grad_a, grad_b, None, None, None, None, None, None, None, None, None


class FP8GroupedGemmTensorFunc(torch.autograd.Function):
    """TENSORWISE grouped GEMM autograd (reference :450-603): one scale per tensor; backward reuses
    the forward's quantized operands."""

    @staticmethod
    def forward(ctx, a, b, a_t, b_t, group_lens, group_offs, trans_b, out_dtype, config, num_cu,
                fuse_bgrad_accum_pattern=None):
        fuse_bgrad_accum, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        assert config.granularity == ScalingGranularity.TENSORWISE
        qa, qa_s, _ = _quantize_plain(a, config, True, -1)
        qb, qb_s, _ = _quantize_plain(b, config, True, -1)
        out = grouped_gemm_fp8_impl(qa, qb, qa_s, qb_s, group_lens, group_offs, False, trans_b, out_dtype,
                                    config.granularity.value, num_cu, _NATIVE)
        if any(ctx.needs_input_grad[:2]):
            ctx.save_for_backward(qa, qb, qa_s, qb_s, group_lens, group_offs)
        ctx.meta = (trans_b, config, out_dtype, num_cu, fuse_bgrad_accum, main_grad)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = _ensure_contiguous_grad_out(grad_out)
        a_q, b_q, a_s, b_s, group_lens, group_offs = ctx.saved_tensors
        trans_b, config, out_dtype, num_cu, fuse_bgrad_accum, main_grad = ctx.meta
        gran = config.granularity.value
        g, g_s, _ = _quantize_plain(grad_out, config, False, -1)
        grad_a = grouped_gemm_fp8_impl(g, b_q, g_s, b_s, group_lens, group_offs, False, not trans_b, out_dtype, gran,
                                       num_cu, _NATIVE)
        grad_b = _grouped_gemm_fp8_variable_k_impl_wrapper(
            a_q, g, a_s, g_s, group_lens, group_offs, True, False, trans_b, out_dtype, gran, num_cu, _NATIVE,
            inplace_add_to_out=fuse_bgrad_accum, out=main_grad,
        )
        return grad_a, grad_b, None, None, None, None, None, None, None, None, None


def _mx_weight_operands(b, b_t, config, need_bwd):
    """The expert weights ``[G, N, K]`` as MXFP8 operands with 32 x 32 blocks: ``(row codes, row scales,
    column codes, column scales)``, the column pair (the transposed quantization dgrad reads) only
    when a backward pass will follow."""
    fdt, bs, gran = _get_fp8_dtype(config.format, True), config.block_size, config.granularity
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
        b_row, b_row_s, b_col, b_col_s = quantize_mxfp8_impl(
            b.contiguous(), fdt, None, bs, with_trans=True, scaling_recipe=w_recipe, scaling_recipe_for_trans=w_recipe)
    else:
        b_row, b_row_s = quantize_mxfp8_impl(b.contiguous(), fdt, 2, bs, scaling_recipe=w_recipe)
    return b_row, b_row_s, b_col, b_col_s


def _mx_backward_products(grad_out, a_col, a_col_s, b_col, b_col_s, group_lens, group_offs, config, dgrad_dtype,
                          wgrad_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad):
    """dgrad and wgrad of the MXFP8 grouped product from the saved column-direction operands."""
    gdt = _get_fp8_dtype(config.format, False)
    gran = config.granularity.value
    g_row, g_row_s, g_col, g_col_s, _, offs_row, lens_col, offs_col = grouped_quantize_mxfp8_impl(
        grad_out, gdt, None, config.block_size, group_lens, group_offs, with_trans=True)
    # dgrad: grad_a = grad_out @ b, as an NT product with the transposed weight quantization [G, K, N]
    grad_a = grouped_gemm_fp8_impl(g_row, b_col, g_row_s, b_col_s, group_lens, offs_row, False, True, dgrad_dtype,
                                   gran, num_cu, _NATIVE, False, group_offs)[:total_m]
    # wgrad: grad_b[g] = grad_out_g^T @ a_g over the 128-padded segments -> [G, N, K]
    grad_b = _grouped_gemm_fp8_variable_k_impl_wrapper(
        g_col, a_col, g_col_s, a_col_s, lens_col, offs_col, False, False, False, wgrad_dtype, gran, num_cu, _NATIVE,
        inplace_add_to_out=fuse_bgrad_accum, out=main_grad,
    )
    return grad_a, grad_b


class FP8GroupedGemmMXFunc(torch.autograd.Function):
    """MX_BLOCKWISE (MXFP8) grouped GEMM autograd."""

    @staticmethod
    def forward(ctx, a, b, a_t, b_t, group_lens, group_offs, trans_b, out_dtype, config, num_cu,
                fuse_bgrad_accum_pattern=None):
        fuse_bgrad_accum, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        assert config.granularity == ScalingGranularity.MX_BLOCKWISE
        assert a.ndim == 2 and b.ndim == 3
        assert trans_b, "MXFP8 grouped GEMM only supports trans_b=True (NT layout)."
        assert group_lens.size(0) == b.size(0), "group_lens size must match b size(0)."
        fdt = _get_fp8_dtype(config.format, True)
        bs = config.block_size
        gran = config.granularity
        total_m = int(a.size(0))
        need_bwd = any(ctx.needs_input_grad[:2])
        a_recipe = ScalingRecipe()
        a_col = a_col_s = None
        if isinstance(a, QuantizedTensor):
            # a grouped (packed rows, per-group padded) quantization made by the caller
            check_quantized_tensor(a, config, axis=-1, scaling_recipe=a_recipe)
            a_row, a_row_s, offs_row = a.qdata, a.scale_inv, a.group_offs
            if need_bwd:
                if a_t is None:
                    a_t = QuantizedTensor.quantize(a.dequantize(), a.real_dtype, gran, axis=-2, block_size=bs,
                                                   scaling_recipe=a_recipe, group_lens=group_lens)
                assert isinstance(a_t, QuantizedTensor)
                a_col, a_col_s = a_t.qdata, a_t.scale_inv
        elif need_bwd:
            a_row, a_row_s, a_col, a_col_s, _, offs_row, _, _ = grouped_quantize_mxfp8_impl(
                a.contiguous(), fdt, None, bs, group_lens, group_offs, with_trans=True)
        else:
            a_row, a_row_s, _, offs_row = grouped_quantize_mxfp8_impl(a.contiguous(), fdt, 1, bs, group_lens, group_offs)
        b_row, b_row_s, b_col, b_col_s = _mx_weight_operands(b, b_t, config, need_bwd)
        # the padded row layout is read through offs_row, the result is packed by group_offs
        # into an output over-allocated to the padded rows
        out = grouped_gemm_fp8_impl(a_row, b_row, a_row_s, b_row_s, group_lens, offs_row, False, True, out_dtype,
                                    config.granularity.value, num_cu, _NATIVE, False, group_offs)[:total_m]
        if need_bwd:
            ctx.save_for_backward(a_col, a_col_s, b_col, b_col_s, group_lens, group_offs)
        ctx.meta = (config, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        grad_out = _ensure_contiguous_grad_out(grad_out)
        a_col, a_col_s, b_col, b_col_s, group_lens, group_offs = ctx.saved_tensors
        config, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad = ctx.meta
        grad_a, grad_b = _mx_backward_products(grad_out, a_col, a_col_s, b_col, b_col_s, group_lens, group_offs, config,
                                               out_dtype, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad)
        return grad_a, grad_b, None, None, None, None, None, None, None, None, None


class FP8GluGroupedGemmMXFunc(torch.autograd.Function):
    """Gated activation -> MXFP8 grouped GEMM (fc2 of an MoE expert MLP) with the activation fused
    into the grouped MX quantizer of the GEMM's activation operand: the bf16 activation is neither
    written nor re-read, forward or backward."""

    @staticmethod
    def forward(ctx, x, probs, row_mask, act_type, b, group_lens, group_offs, trans_b, out_dtype, config, num_cu,
                fuse_bgrad_accum_pattern=None):
        fuse_bgrad_accum, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        assert config.granularity == ScalingGranularity.MX_BLOCKWISE and config.block_size == 32
        assert x.ndim == 2 and x.size(1) % 2 == 0, "x must be [tokens, 2 * hidden]"
        assert trans_b, "MXFP8 grouped GEMM only supports trans_b=True (NT layout)."
        assert group_lens.size(0) == b.size(0), "group_lens size must match b size(0)."
        assert probs.dtype == torch.float32 and probs.numel() == x.size(0), "probs must be float32, one per token"
        total_m = int(x.size(0))
        need_bwd = any(ctx.needs_input_grad[i] for i in (0, 1, 4))
        x2, p1 = x.contiguous(), probs.reshape(-1).contiguous()
        a_row, a_row_s, a_col, a_col_s, _, offs_row, _, _ = glu_grouped_quantize_mx_impl(
            x2, p1, row_mask, act_type, _get_fp8_dtype(config.format, True), group_lens, group_offs, need_bwd)
        b_row, b_row_s, b_col, b_col_s = _mx_weight_operands(b, None, config, need_bwd)
        out = grouped_gemm_fp8_impl(a_row, b_row, a_row_s, b_row_s, group_lens, offs_row, False, True, out_dtype,
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
        grad_act, grad_b = _mx_backward_products(grad_out, a_col, a_col_s, b_col, b_col_s, group_lens, group_offs, config,
                                                 x2.dtype, out_dtype, num_cu, total_m, fuse_bgrad_accum, main_grad)
        grad_x, grad_probs = glu_bwd_with_probs(grad_act.contiguous(), x2, p1, row_mask,
                                                ACT_SILU if act_type == "silu" else ACT_GELU)
        return grad_x, grad_probs.view(probs_shape), None, None, grad_b, None, None, None, None, None, None, None


def grouped_gemm_fp8(
    a: Union[torch.Tensor, QuantizedTensor, QuantizedTensorPair],
    b: Union[torch.Tensor, QuantizedTensor, QuantizedTensorPair],
    group_lens: torch.Tensor,
    group_offs: Optional[torch.Tensor] = None,
    trans_b: bool = True,
    out_dtype: Optional[torch.dtype] = None,
    config: Optional[Float8QuantConfig] = None,
    num_cu: Optional[int] = None,
    fuse_bgrad_accum_pattern: Optional[str] = None,
) -> torch.Tensor:
    """Grouped GEMM with FP8 quantization: ``out[rows of group g] = a[rows of group g] @ op(b[g])``.

    ``a``: ``[sum(group_lens), k]`` (fp16 / bf16); ``b``: ``[G, n, k]`` if ``trans_b`` else
    ``[G, k, n]`` (or a pre-quantized 2-D-block ``QuantizedTensor``); ``group_lens``: int64 ``[G]``
    on the device (groups may be empty); ``config``: BLOCKWISE with ``block_size=128``."""
    if config is None:
        config = Float8QuantConfig()
    if group_offs is None:
        group_offs = group_offs_from_lens(group_lens)
    a_data, a_data_t = (a.data, a.data_t) if isinstance(a, QuantizedTensorPair) else (a, None)
    b_data, b_data_t = (b.data, b.data_t) if isinstance(b, QuantizedTensorPair) else (b, None)
    if out_dtype is None:
        out_dtype = torch.promote_types(a_data.dtype, b_data.dtype)
    if config.granularity == ScalingGranularity.BLOCKWISE:
        return FP8GroupedGemmBlockFunc.apply(a_data, b_data, a_data_t, b_data_t, group_lens, group_offs, trans_b,
                                             out_dtype, config, num_cu, fuse_bgrad_accum_pattern)
    if config.granularity == ScalingGranularity.ROWWISE:
        return FP8GroupedGemmRowFunc.apply(a_data, b_data, a_data_t, b_data_t, group_lens, group_offs, trans_b,
                                           out_dtype, config, num_cu, fuse_bgrad_accum_pattern)
    if config.granularity == ScalingGranularity.TENSORWISE:
        return FP8GroupedGemmTensorFunc.apply(a_data, b_data, a_data_t, b_data_t, group_lens, group_offs, trans_b,
                                              out_dtype, config, num_cu, fuse_bgrad_accum_pattern)
    if config.granularity == ScalingGranularity.MX_BLOCKWISE:
        return FP8GroupedGemmMXFunc.apply(a_data, b_data, a_data_t, b_data_t, group_lens, group_offs, trans_b,
                                          out_dtype, config, num_cu, fuse_bgrad_accum_pattern)
    raise NotImplementedError(
        f"grouped_gemm_fp8: unknown granularity {config.granularity}"
    )


def glu_grouped_gemm_fp8(
    x: torch.Tensor,
    probs: torch.Tensor,
    b: Union[torch.Tensor, QuantizedTensor],
    group_lens: torch.Tensor,
    group_offs: Optional[torch.Tensor] = None,
    trans_b: bool = True,
    out_dtype: Optional[torch.dtype] = None,
    config: Optional[Float8QuantConfig] = None,
    num_cu: Optional[int] = None,
    row_mask: Optional[torch.Tensor] = None,
    act_type: str = "silu",
    fuse_bgrad_accum_pattern: Optional[str] = None,
) -> torch.Tensor:
    """``grouped_gemm_fp8(swiglu_with_probs(x, probs, row_mask), b, group_lens, ...)`` (``act_type="gelu"``:
    ``geglu_with_probs``) as one operation for the BLOCKWISE and MX_BLOCKWISE configurations: fc1's output ``x [tokens, 2 H]``
    is read once by a quantizer that applies the gated activation on load, so the bf16 activation
    never goes through HBM; results and gradients are bit-identical with the two-step form when ``x``, ``b`` and
    ``out_dtype`` are one type (otherwise the activation gradient is written in ``x``'s type directly). (The
    reference has the two steps only: ops/activation.py:21-83, ops/grouped_gemm_fp8.py:99-265.)"""
    if config is None:
        config = Float8QuantConfig(granularity=ScalingGranularity.BLOCKWISE, block_size=128)
    if config.granularity not in (ScalingGranularity.BLOCKWISE, ScalingGranularity.MX_BLOCKWISE):
        raise NotImplementedError(
            "glu_grouped_gemm_fp8: the fused quantizer exists for the BLOCKWISE and MX_BLOCKWISE configurations")
    assert act_type in ("silu", "gelu"), f"Unsupported act_type: {act_type}"
    if group_offs is None:
        group_offs = group_offs_from_lens(group_lens)
    if out_dtype is None:
        out_dtype = torch.promote_types(x.dtype, b.dtype)
    if config.granularity == ScalingGranularity.MX_BLOCKWISE:
        return FP8GluGroupedGemmMXFunc.apply(x, probs, row_mask, act_type, b, group_lens, group_offs, trans_b, out_dtype,
                                             config, num_cu, fuse_bgrad_accum_pattern)
    return FP8GluGroupedGemmBlockFunc.apply(x, probs, row_mask, act_type, b, group_lens, group_offs, trans_b, out_dtype,
                                            config, num_cu, fuse_bgrad_accum_pattern)
