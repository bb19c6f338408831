"""``gemm_fp8``: FP8 GEMM with autograd (reference: primus_turbo/pytorch/ops/gemm_fp8.py).

Which quantizer feeds which GEMM layout, per granularity (same recipes as the reference):

  TENSORWISE  fwd  C = Aq . Bq            one scale per tensor; backward runs NT GEMMs on
                   physically transposed fp8 copies when the forward is NT (ref :96-276)
  ROWWISE     fwd  A, B quantized along K; backward re-quantizes the de-quantized
                   operands along the other axis and quantizes grad_out twice (ref :278-426)
  BLOCKWISE   fwd  A 1x128 (+128x1 for wgrad from the same read), B 128x128 tiles;
                   dgrad = NN with the same weight tiles, wgrad = TN on the 128x1 casts
                   (ref :429-553)
  MX_BLOCKWISE     A 1x32, B 32x32 two-direction MXFP8 casts, every GEMM is NT (ref :556-717)

HYBRID format: forward operands E4M3, gradients E5M2.
"""

from __future__ import annotations

from typing import Optional, Union

import torch

from primus_turbo.pytorch.core.backend import BackendType
from primus_turbo.pytorch.core.low_precision import (
    Float8QuantConfig,
    ScalingGranularity,
    ScalingRecipe,
    check_mxfp8_support,
)
from primus_turbo.pytorch.core.quantized_tensor import (
    QuantizedTensor,
    QuantizedTensorPair,
    check_quantized_tensor,
    transpose_last_two,
)
from primus_turbo.pytorch.kernels.gemm.gemm_fp8_impl import gemm_fp8_accum_impl, gemm_fp8_impl
from primus_turbo.pytorch.kernels.quantization.quantization_impl import (
    quant_fp8_blockwise_dual_t_impl,
    quant_fp8_blockwise_kmajor_impl,
    quant_fp8_blockwise_for_weight_dual_impl,
)
from primus_turbo.pytorch.ops.quantization import dequantize_fp8, quantize_fp8, quantize_fp8_with_trans
from primus_turbo.pytorch.ops.utils import _get_dummy_wgrad, _get_fp8_dtype, _setup_fused_grad_accum

__all__ = ["gemm_fp8"]

_NATIVE = BackendType.TURBO.value  # single backend; the value is informational


def _gemm(a, a_s, trans_a, b, b_s, trans_b, out_dtype, trans_c, granularity):
    return gemm_fp8_impl(a, a_s, trans_a, b, b_s, trans_b, out_dtype, trans_c, granularity.value, _NATIVE)


def _wgrad_gemm(a, a_s, trans_a, b, b_s, trans_b, out_dtype, trans_c, granularity, accumulate_into=None):
    """Weight-gradient GEMM; with ``accumulate_into`` the result is added to that buffer in
    the GEMM epilogue and a cached dummy tensor of the weight's shape is returned (the
    framework's own accumulation was switched off in forward)."""
    if accumulate_into is None:
        return _gemm(a, a_s, trans_a, b, b_s, trans_b, out_dtype, trans_c, granularity)
    gemm_fp8_accum_impl(a, a_s, trans_a, b, b_s, trans_b, accumulate_into.dtype, trans_c, granularity.value,
                        accumulate_into, _NATIVE)
    return _get_dummy_wgrad(accumulate_into.shape, out_dtype)


def _quantized_parts(x, config, fwd: bool, axis):
    """-> ``(codes, scale_inv, original dtype)`` of an operand: the fields of a ``QuantizedTensor``
    that the caller quantized already, else a fresh quantization along ``axis``. Plain tensors, not
    wrappers, so that ``torch.compile`` traces the functions below into one graph."""
    if isinstance(x, QuantizedTensor):
        check_quantized_tensor(x, config, axis=axis)
        return x.qdata, x.scale_inv, x.dtype
    q, s = quantize_fp8(x.contiguous(), _get_fp8_dtype(config.format, fwd), config.granularity, axis=axis % x.ndim,
                        block_size=config.block_size)
    return q, s, x.dtype


class FP8GemmTensorFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, a_t, b_t, trans_a, trans_b, out_dtype, config, fuse_bgrad_accum_pattern=None):
        fuse, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        qa, qa_s, _ = _quantized_parts(a, config, True, -1)
        qb, qb_s, _ = _quantized_parts(b, config, True, -1)
        out = _gemm(qa, qa_s, trans_a, qb, qb_s, trans_b, out_dtype, False, config.granularity)
        # NT forward: keep physically transposed fp8 copies so that both backward GEMMs
        # are NT as well (contiguous-K operands need no transposition pass inside the GEMM)
        nt_bwd = (not trans_a) and trans_b
        if nt_bwd:
            # a tensorwise transpose moves the codes and shares the scalar scale
            sa, sa_s = (a_t.qdata, a_t.scale_inv) if isinstance(a_t, QuantizedTensor) else (transpose_last_two(qa), qa_s)
            sb, sb_s = (b_t.qdata, b_t.scale_inv) if isinstance(b_t, QuantizedTensor) else (transpose_last_two(qb), qb_s)
            ctx.save_for_backward(sa, sa_s, sb, sb_s)
        else:
            ctx.save_for_backward(qa, qa_s, qb, qb_s)
        ctx.meta = (trans_a, trans_b, out_dtype, config, nt_bwd, fuse, main_grad)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        trans_a, trans_b, out_dtype, config, nt_bwd, fuse, main_grad = ctx.meta
        sa, sa_s, sb, sb_s = ctx.saved_tensors
        gran = config.granularity
        g, g_s = quantize_fp8(grad_out.contiguous(), _get_fp8_dtype(config.format, False), gran)
        acc = main_grad if fuse else None
        if nt_bwd:
            # saved: A^T [K, M], B^T [K, N]
            grad_a = _gemm(g, g_s, False, sb, sb_s, True, out_dtype, False, gran)
            grad_b = _wgrad_gemm(sa, sa_s, False, transpose_last_two(g), g_s, True, out_dtype, trans_b, gran, acc)
        else:
            grad_a = _gemm(g, g_s, False, sb, sb_s, not trans_b, out_dtype, trans_a, gran)
            grad_b = _wgrad_gemm(sa, sa_s, not trans_a, g, g_s, False, out_dtype, trans_b, gran, acc)
        return grad_a, grad_b, None, None, None, None, None, None, None


class FP8GemmRowFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, a_t, b_t, trans_a, trans_b, out_dtype, config):
        assert trans_a == False, "trans_a has to be False"  # noqa: E712
        gran = config.granularity
        b_axis = -1 if trans_b else -2
        qa, qa_s, a_hp = _quantized_parts(a, config, True, -1)
        qb, qb_s, b_hp = _quantized_parts(b, config, True, b_axis)

        def other_axis(q, q_s, hp_dtype, from_axis, given, axis):
            # the operand as backward reads it: what the forward codes stand for, quantized again
            # along the other axis
            if given is not None:
                assert isinstance(given, QuantizedTensor)
                return given.qdata, given.scale_inv
            hp = dequantize_fp8(q, hp_dtype, gran, axis=from_axis % q.ndim, scale_inv=q_s, block_size=config.block_size)
            return quantize_fp8(hp, q.dtype, gran, axis=axis % q.ndim, block_size=config.block_size)

        out = _gemm(qa, qa_s, trans_a, qb, qb_s, trans_b, out_dtype, False, gran)
        # the operands quantized along their other axis only feed backward: skip them when no
        # input asks for a gradient (same outputs, two quantizer passes less)
        if any(ctx.needs_input_grad[:2]):
            a_c, a_cs = other_axis(qa, qa_s, a_hp, -1, a_t, -2)
            b_c, b_cs = other_axis(qb, qb_s, b_hp, b_axis, b_t, -2 if trans_b else -1)
            ctx.save_for_backward(a_c, a_cs, b_c, b_cs)
        ctx.meta = (trans_a, trans_b, out_dtype, config)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        trans_a, trans_b, out_dtype, config = ctx.meta
        a_c, a_cs, b_c, b_cs = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        gdt = _get_fp8_dtype(config.format, False)
        gran = config.granularity
        g_row, g_row_s = quantize_fp8(grad_out, gdt, gran, axis=1, block_size=config.block_size)
        grad_a = _gemm(g_row, g_row_s, False, b_c, b_cs, not trans_b, out_dtype, trans_a, gran)
        g_col, g_col_s = quantize_fp8(grad_out, gdt, gran, axis=0, block_size=config.block_size)
        grad_b = _gemm(a_c, a_cs, not trans_a, g_col, g_col_s, False, out_dtype, trans_b, gran)
        return grad_a, grad_b, None, None, None, None, None, None


class FP8GemmBlockFunction(torch.autograd.Function):
    """BLOCKWISE (128): activations and gradients in 1 x 128 blocks along the reduction of each
    product, the weight in 128 x 128 tiles that serve forward and backward. When a gradient is
    wanted the quantizers also emit, from the same read, the operands of the backward products with
    their reduction axis contiguous (the transposed 128 x 1 column codes of ``a`` and ``grad_out``,
    the transposed weight codes), so that every product is an NT product read in place."""

    @staticmethod
    def forward(ctx, a, b, a_t, b_t, trans_a, trans_b, out_dtype, config):
        assert trans_a == False, "trans_a has to be False"  # noqa: E712
        fdt = _get_fp8_dtype(config.format, True)
        gran, bs = config.granularity, config.block_size
        need_bwd = any(ctx.needs_input_grad[:2])
        a_col = a_col_s = None
        a_kmajor = False
        if isinstance(a, QuantizedTensor):
            check_quantized_tensor(a, config, axis=-1)
            a_row, a_row_s = a.qdata, a.scale_inv
            if need_bwd:
                if a_t is None:
                    a_t = QuantizedTensor.quantize(a.dequantize(), fdt, gran, axis=-2, block_size=bs)
                a_col, a_col_s = a_t.qdata, a_t.scale_inv
        elif a.dim() == 2:
            # row scales block-major, as the GEMM reads them; the column-direction copy of `a` only
            # feeds wgrad: skipped when nothing asks for a gradient
            a_row, a_row_s_km, a_col, a_col_s = quant_fp8_blockwise_kmajor_impl(a.contiguous(), fdt, bs, need_bwd)
            a_row_s = a_row_s_km.t()
            a_kmajor = need_bwd
        else:
            a_row, a_row_s = quantize_fp8(a, fdt, gran, axis=-1, block_size=bs)
        w_recipe = ScalingRecipe(use_2d_block=True)  # weight tiles serve forward and backward unchanged
        b_q_t = None
        if isinstance(b, QuantizedTensor):
            check_quantized_tensor(b, config, scaling_recipe=w_recipe)
            b_q, b_s = b.qdata, b.scale_inv
        elif (need_bwd or not trans_b) and b.dim() == 2 and b.size(0) % 16 == 0:
            b_q, b_q_t, b_s = quant_fp8_blockwise_for_weight_dual_impl(b, fdt, bs)
        else:
            b_q, b_s = quantize_fp8(b, fdt, gran, block_size=bs, scaling_recipe=w_recipe)
        b_s_t = b_s.t().contiguous() if b_q_t is not None else None
        # forward reduces over b's last axis when trans_b, dgrad over the other one
        fwd_b, fwd_s, dgrad_b, dgrad_s = (b_q, b_s, b_q_t, b_s_t) if trans_b else (b_q_t, b_s_t, b_q, b_s)
        if fwd_b is not None:
            out = _gemm(a_row, a_row_s, False, fwd_b, fwd_s, True, out_dtype, False, gran)
        else:
            out = _gemm(a_row, a_row_s, False, b_q, b_s, trans_b, out_dtype, False, gran)
        if need_bwd:
            b_ready = dgrad_b is not None
            ctx.save_for_backward(a_col, a_col_s, dgrad_b if b_ready else b_q, dgrad_s if b_ready else b_s)
            ctx.meta = (trans_a, trans_b, out_dtype, config, a_kmajor, b_ready)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        trans_a, trans_b, out_dtype, config, a_kmajor, b_ready = ctx.meta
        a_col, a_col_s, b_q, b_s = ctx.saved_tensors
        gran = config.granularity
        gdt = _get_fp8_dtype(config.format, False)
        g = grad_out.contiguous()
        if a_kmajor:
            g_row, g_row_s_km, g_col_t, g_col_s = quant_fp8_blockwise_kmajor_impl(g, gdt, config.block_size, True)
            g_row_s = g_row_s_km.t()
        else:
            g_row, g_row_s, g_col, g_col_s = quantize_fp8_with_trans(g, gdt, gran, block_size=config.block_size)
        grad_a = _gemm(g_row, g_row_s, False, b_q, b_s, True if b_ready else not trans_b, out_dtype, False, gran)
        if a_kmajor:
            # [K, M_pad] x [N, M_pad]^T: both read in place; trans_c gives the [N, K] weight layout
            grad_b = _gemm(a_col, a_col_s, False, g_col_t, g_col_s, True, out_dtype, trans_b, gran)
        else:
            grad_b = _gemm(a_col, a_col_s, not trans_a, g_col, g_col_s, False, out_dtype, trans_b, gran)
        return grad_a, grad_b, None, None, None, None, None, None


class FP8GemmMXFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, a_t, b_t, trans_a, trans_b, out_dtype, config, fuse_bgrad_accum_pattern=None):
        from primus_turbo.pytorch.kernels.quantization.quantization_impl import quantize_mxfp8_impl

        ok, why = check_mxfp8_support()
        assert ok, why
        assert trans_a == False and trans_b == True, "trans_a has to be False and trans_b has to be True"  # noqa: E712
        fuse, main_grad = _setup_fused_grad_accum(b, fuse_bgrad_accum_pattern)
        fdt = _get_fp8_dtype(config.format, True)
        gran, bs = config.granularity, config.block_size

        need_bwd = any(ctx.needs_input_grad[:2])

        def both_ways(x, x_t, recipe):
            if isinstance(x, QuantizedTensor):
                check_quantized_tensor(x, config, axis=-1, scaling_recipe=recipe)
                if x_t is None:
                    x_t = QuantizedTensor.quantize(x.dequantize(), x.real_dtype, gran, axis=-2, block_size=bs,
                                                   scaling_recipe=recipe)
                return x.qdata, x.scale_inv, x_t.qdata, x_t.scale_inv
            if not need_bwd:
                # the transposed copies only feed backward: skip them when nothing asks for a gradient
                q, sc = quantize_mxfp8_impl(x, fdt, x.dim() - 1, bs, scaling_recipe=recipe)
                return q, sc, q, sc
            return quantize_mxfp8_impl(x, fdt, None, bs, with_trans=True, scaling_recipe=recipe,
                                       scaling_recipe_for_trans=recipe)

        a_row, a_row_s, a_col, a_col_s = both_ways(a, a_t, ScalingRecipe())
        b_row, b_row_s, b_col, b_col_s = both_ways(b, b_t, ScalingRecipe(use_2d_block=True))
        out = _gemm(a_row, a_row_s, False, b_row, b_row_s, True, out_dtype, False, gran)
        ctx.save_for_backward(a_col, a_col_s, b_col, b_col_s)
        ctx.meta = (out_dtype, config, fuse, main_grad)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        from primus_turbo.pytorch.kernels.quantization.quantization_impl import quantize_mxfp8_impl

        out_dtype, config, fuse, main_grad = ctx.meta
        a_col, a_col_s, b_col, b_col_s = ctx.saved_tensors
        gran = config.granularity
        g = grad_out.reshape(grad_out.shape[0], -1).contiguous()
        g_row, g_row_s, g_col, g_col_s = quantize_mxfp8_impl(
            g, _get_fp8_dtype(config.format, False), None, config.block_size, with_trans=True,
            scaling_recipe=ScalingRecipe(), scaling_recipe_for_trans=ScalingRecipe(),
        )
        # the two-direction casts are stored transposed, so dgrad and wgrad are NT GEMMs too
        grad_a = _gemm(g_row, g_row_s, False, b_col, b_col_s, True, out_dtype, False, gran)
        grad_b = _wgrad_gemm(g_col, g_col_s, False, a_col, a_col_s, True, out_dtype, False, gran,
                             main_grad if fuse else None)
        return grad_a, grad_b, None, None, None, None, None, None, None


def gemm_fp8(
    a: Union[torch.Tensor, QuantizedTensor, QuantizedTensorPair],
    b: Union[torch.Tensor, QuantizedTensor, QuantizedTensorPair],
    trans_a: bool = False,
    trans_b: bool = False,
    out_dtype: Optional[torch.dtype] = None,
    config: Optional[Float8QuantConfig] = None,
    fuse_bgrad_accum_pattern: Optional[str] = None,
) -> torch.Tensor:
    """FP8 GEMM with autograd: ``a`` is ``(M, K)``, ``b`` is ``(K, N)`` or, with
    ``trans_b``, ``(N, K)``; returns ``(M, N)`` in ``out_dtype``.

    ``config`` selects format (E4M3 / E5M2 / HYBRID) and granularity (TENSORWISE default,
    ROWWISE, BLOCKWISE with ``block_size=128``, MX_BLOCKWISE with ``block_size=32`` and E8M0
    scales). Operands may be pre-quantized ``QuantizedTensor`` / ``QuantizedTensorPair``.
    ``fuse_bgrad_accum_pattern="megatron"`` (TENSORWISE and MX_BLOCKWISE) adds the weight
    gradient into ``b.main_grad`` inside the wgrad GEMM epilogue.
    """
    if config is None:
        config = Float8QuantConfig()
    a_data, a_t = (a.data, a.data_t) if isinstance(a, QuantizedTensorPair) else (a, None)
    b_data, b_t = (b.data, b.data_t) if isinstance(b, QuantizedTensorPair) else (b, None)
    assert a_data.ndim == 2, "Only 2D tensors are supported"
    assert b_data.ndim == 2, "Only 2D tensors are supported"
    if out_dtype is None:
        out_dtype = torch.promote_types(a_data.dtype, b_data.dtype)

    g = config.granularity
    if g == ScalingGranularity.TENSORWISE:
        return FP8GemmTensorFunction.apply(a_data, b_data, a_t, b_t, trans_a, trans_b, out_dtype, config,
                                           fuse_bgrad_accum_pattern)
    if g == ScalingGranularity.MX_BLOCKWISE:
        return FP8GemmMXFunction.apply(a_data, b_data, a_t, b_t, trans_a, trans_b, out_dtype, config,
                                       fuse_bgrad_accum_pattern)
    assert fuse_bgrad_accum_pattern is None, f"fuse_bgrad_accum_pattern is not supported for {g}"
    if g == ScalingGranularity.ROWWISE:
        return FP8GemmRowFunction.apply(a_data, b_data, a_t, b_t, trans_a, trans_b, out_dtype, config)
    if g == ScalingGranularity.BLOCKWISE:
        return FP8GemmBlockFunction.apply(a_data, b_data, a_t, b_t, trans_a, trans_b, out_dtype, config)
    raise ValueError(f"Unsupported FP8 ScalingGranularity: {g}")
