"""MXFP4 GEMM impl layer: the reference's ``gemm_fp4_impl`` / ``gemm_fp4_accum_impl`` contracts
(primus_turbo/pytorch/kernels/gemm/gemm_fp4_impl.py:339-430 of the reference) on ``pt_gemm_mx``.

NT layout only, as in the reference (its hipBLASLt / AITER backends support nothing else);
``default_backend`` is accepted and ignored. ``preshuffled`` operands (the layout the reference hands
to AITER, its lines 197-211: ``a`` plain codes with shuffled scales, ``b`` shuffled codes and scales)
are brought back to the plain layout by two small passes before the product: the kernel here reads
row-major operands at full rate, so nothing is gained by holding weights pre-shuffled.
"""

from __future__ import annotations

import torch

from primus_turbo.pytorch.core.low_precision import ScalingGranularity
from primus_turbo.pytorch.kernels.gemm.gemm_fp8_impl import _check, launch_mx


def _plain_operands(a, a_scale_inv, b, b_scale_inv, preshuffled):
    if not preshuffled:
        return a, a_scale_inv, b, b_scale_inv
    from primus_turbo.pytorch.kernels.quantization.quantization_impl import mx_plain_layout

    a, a_scale_inv = mx_plain_layout(a, a_scale_inv, False, True)
    b, b_scale_inv = mx_plain_layout(b, b_scale_inv, True, True)
    return a, a_scale_inv, b, b_scale_inv


def _validate(a, trans_a, b, trans_b, granularity, preshuffled):
    _check(ScalingGranularity(granularity) == ScalingGranularity.MX_BLOCKWISE, "gemm_fp4 supports MX_BLOCKWISE only")
    _check(not trans_a and trans_b, "MXFP4 GEMM supports the NT layout only (trans_a=False, trans_b=True)")
    fp4 = getattr(torch, "float4_e2m1fn_x2", None)
    _check(fp4 is not None and a.dtype == fp4 and b.dtype == fp4, "operands must be float4_e2m1fn_x2")


@torch.library.custom_op("primus_turbo::gemm_fp4_impl", mutates_args=(), device_types="cuda")
def gemm_fp4_impl(
    a: torch.Tensor,
    a_scale_inv: torch.Tensor,
    trans_a: bool,
    b: torch.Tensor,
    b_scale_inv: torch.Tensor,
    trans_b: bool,
    out_dtype: torch.dtype,
    trans_c: bool,
    granularity: int,
    default_backend: int,
    preshuffled: bool = False,
) -> torch.Tensor:
    """``out = a @ b.T`` for MXFP4 operands ``a [M, K/2]``, ``b [N, K/2]`` (two E2M1 codes per
    byte) with E8M0 scales ``[rows, K/32]``; ``trans_c`` returns the transposed product."""
    _validate(a, trans_a, b, trans_b, granularity, preshuffled)
    a, a_scale_inv, b, b_scale_inv = _plain_operands(a, a_scale_inv, b, b_scale_inv, preshuffled)
    M, Nn = a.shape[0], b.shape[0]
    out = torch.empty((Nn, M) if trans_c else (M, Nn), dtype=out_dtype, device=a.device)
    return launch_mx(a, a_scale_inv, b, b_scale_inv, out, trans_c, False)


@gemm_fp4_impl.register_fake
def _gemm_fp4_impl_fake(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out_dtype, trans_c, granularity,
                        default_backend, preshuffled=False):
    M, Nn = a.shape[0], b.shape[0]
    return torch.empty((Nn, M) if trans_c else (M, Nn), dtype=out_dtype, device=a.device)


@torch.library.custom_op("primus_turbo::gemm_fp4_accum_impl", mutates_args={"out"}, device_types="cuda")
def gemm_fp4_accum_impl(
    a: torch.Tensor,
    a_scale_inv: torch.Tensor,
    trans_a: bool,
    b: torch.Tensor,
    b_scale_inv: torch.Tensor,
    trans_b: bool,
    out_dtype: torch.dtype,
    trans_c: bool,
    granularity: int,
    out: torch.Tensor,
    default_backend: int,
    preshuffled: bool = False,
) -> None:
    """Same product added into ``out`` (beta = 1 in the GEMM epilogue)."""
    _validate(a, trans_a, b, trans_b, granularity, preshuffled)
    a, a_scale_inv, b, b_scale_inv = _plain_operands(a, a_scale_inv, b, b_scale_inv, preshuffled)
    launch_mx(a, a_scale_inv, b, b_scale_inv, out, trans_c, True)


@gemm_fp4_accum_impl.register_fake
def _gemm_fp4_accum_impl_fake(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out_dtype, trans_c, granularity, out,
                              default_backend, preshuffled=False):
    return None
