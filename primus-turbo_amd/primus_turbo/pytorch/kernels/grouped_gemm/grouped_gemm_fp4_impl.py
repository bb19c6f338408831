"""Grouped MXFP4 GEMM operators: the ``grouped_gemm_fp4_impl`` / ``grouped_gemm_fp4_variable_k_impl``
/ ``..._variable_k_accum_impl`` contracts (reference:
primus_turbo/pytorch/kernels/grouped_gemm/grouped_gemm_fp4_impl.py:429-560) on the gfx950 MX
kernel: packed E2M1 operands, one E8M0 scale per 32 elements of K applied by the matrix core.

Forward / dgrad multiply the tight rows of every group with the group's ``[N, K]`` weight;
wgrad reduces over each group's 256-padded token range of the transposed column-direction
operands. The backend arguments are accepted and ignored: a single implementation exists."""

from __future__ import annotations

from typing import Optional

import torch

from primus_turbo.pytorch.core.low_precision import ScalingGranularity
from primus_turbo.pytorch.kernels.grouped_gemm.grouped_gemm_fp8_impl import _grouped_mx, _variable_k_mx

_FP4X2 = getattr(torch, "float4_e2m1fn_x2", None)


def _check_mx(granularity: int, *ts) -> None:
    if ScalingGranularity(granularity) != ScalingGranularity.MX_BLOCKWISE:
        raise ValueError(f"Unsupported FP4 ScalingGranularity: {ScalingGranularity(granularity)}")
    for t in ts:
        if _FP4X2 is None or t.dtype != _FP4X2:
            raise RuntimeError(f"operands must be float4_e2m1fn_x2, got {t.dtype}")


@torch.library.custom_op("primus_turbo::grouped_gemm_fp4_impl", mutates_args=(), device_types="cuda")
def grouped_gemm_fp4_impl(
    a: torch.Tensor,
    b: torch.Tensor,
    a_scales: torch.Tensor,
    b_scales: torch.Tensor,
    group_lens: torch.Tensor,
    group_offs: torch.Tensor,
    trans_a: bool,
    trans_b: bool,
    out_dtype: torch.dtype,
    granularity: int,
    num_cu: Optional[int],
    default_backend: int,
    maybe_pre_sync: bool = False,
    group_offs_out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``out[oo[g]:oo[g+1]] = a[o[g] : o[g] + len_g] @ b[g]^T``; rows past ``oo[G]`` are zero.

    ``a`` ``[rows, K/2]`` packed codes with scales ``[rows, K/32]``, ``b`` ``[G, N, K/2]`` with
    ``[G, N, K/32]``; ``o`` = ``group_offs``, ``oo`` = ``group_offs_out`` (default ``o``)."""
    _check_mx(granularity, a, b)
    return _grouped_mx(a, b, a_scales, b_scales, group_offs, group_offs_out, trans_a, trans_b, out_dtype)


@grouped_gemm_fp4_impl.register_fake
def _grouped_gemm_fp4_impl_fake(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b, out_dtype,
                                granularity, num_cu, default_backend, maybe_pre_sync=False, group_offs_out=None):
    assert a.dim() == 2, f"a must be 2D, got {a.shape}"
    assert b.dim() == 3, f"b must be 3D, got {b.shape}"
    assert not trans_a, "Only trans_a=False is supported."
    return torch.empty((a.shape[0], b.shape[-2] if trans_b else b.shape[-1]), device=a.device, dtype=out_dtype)


def _variable_k_out(a, b, group_offs, trans_c, out_dtype):
    G = group_offs.numel() - 1
    Ml, Nr = (b.shape[0], a.shape[0]) if trans_c else (a.shape[0], b.shape[0])
    return torch.empty((G, Ml, Nr), dtype=out_dtype, device=a.device)


@torch.library.custom_op("primus_turbo::grouped_gemm_fp4_variable_k_impl", mutates_args=(), device_types="cuda")
def grouped_gemm_fp4_variable_k_impl(
    a: torch.Tensor,
    b: torch.Tensor,
    a_scales: torch.Tensor,
    b_scales: torch.Tensor,
    group_lens: torch.Tensor,
    group_offs: torch.Tensor,
    trans_a: bool,
    trans_b: bool,
    trans_c: bool,
    out_dtype: torch.dtype,
    granularity: int,
    num_cu: Optional[int],
    default_backend: int,
    maybe_pre_sync: bool = False,
) -> torch.Tensor:
    """``out[g] = a[:, p[g]:p[g+1]] @ b[:, p[g]:p[g+1]]^T`` (transposed when ``trans_c``) with
    ``a`` ``[Ml, M_pad/2]`` and ``b`` ``[Nr, M_pad/2]`` the transposed column-direction outputs of
    the grouped quantizer and ``p`` = ``group_offs`` their 256-padded offsets in elements."""
    _check_mx(granularity, a, b)
    out = _variable_k_out(a, b, group_offs, trans_c, out_dtype)
    return _variable_k_mx(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, False)


@grouped_gemm_fp4_variable_k_impl.register_fake
def _grouped_gemm_fp4_variable_k_impl_fake(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b, trans_c,
                                           out_dtype, granularity, num_cu, default_backend, maybe_pre_sync=False):
    assert a.dim() == 2 and b.dim() == 2
    return _variable_k_out(a, b, group_offs, trans_c, out_dtype)


@torch.library.custom_op("primus_turbo::grouped_gemm_fp4_variable_k_accum_impl", mutates_args={"out"},
                         device_types="cuda")
def grouped_gemm_fp4_variable_k_accum_impl(
    a: torch.Tensor,
    b: torch.Tensor,
    a_scales: torch.Tensor,
    b_scales: torch.Tensor,
    group_lens: torch.Tensor,
    group_offs: torch.Tensor,
    trans_a: bool,
    trans_b: bool,
    trans_c: bool,
    out_dtype: torch.dtype,
    granularity: int,
    num_cu: Optional[int],
    default_backend: int,
    out: torch.Tensor,
    maybe_pre_sync: bool = False,
) -> None:
    """As ``grouped_gemm_fp4_variable_k_impl`` with ``out[g] +=`` folded into the epilogue
    (``out`` may be fp32, bf16 or fp16)."""
    _check_mx(granularity, a, b)
    _variable_k_mx(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, True)


@grouped_gemm_fp4_variable_k_accum_impl.register_fake
def _grouped_gemm_fp4_variable_k_accum_impl_fake(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b,
                                                 trans_c, out_dtype, granularity, num_cu, default_backend, out,
                                                 maybe_pre_sync=False):
    assert a.dim() == 2 and b.dim() == 2 and out.dim() == 3
    return None
