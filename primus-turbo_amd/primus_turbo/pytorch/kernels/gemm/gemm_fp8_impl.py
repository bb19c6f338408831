"""Dense FP8 GEMM impl layer: maps the reference's ``gemm_fp8_impl`` contract
(primus_turbo/pytorch/kernels/gemm/gemm_fp8_impl.py:518-633 of the reference) onto the
single gfx950 kernel family behind ``pt_gemm_fp8``.

The reference dispatches among five backends; here there is one, so ``default_backend``
is accepted and ignored. What this layer owns is the translation of each granularity's
scale tensors and operand layouts into the kernel's (stride, block) description.
"""

from __future__ import annotations

from typing import Tuple

import torch

from primus_turbo import _native as N
from primus_turbo.pytorch.core.low_precision import ScalingGranularity

_FP8 = (torch.float8_e4m3fn, torch.float8_e5m2)
_OUT = (torch.bfloat16, torch.float16, torch.float32)

TILE_CFG = 0  # 0 = automatic; tests and the benchmark may pin 1 (256x256), 2 (256x128), 3 (128x128), 4 (256x256, eight wavefronts: block scales)


def get_gemm_logical_shape(a: torch.Tensor, b: torch.Tensor, trans_a: bool, trans_b: bool) -> Tuple[int, int, int]:
    assert a.dim() == 2 and b.dim() == 2, "gemm_fp8 expects 2-D operands"
    M, K = (a.shape[1], a.shape[0]) if trans_a else a.shape
    Kb, Nn = (b.shape[1], b.shape[0]) if trans_b else b.shape
    assert K == Kb, f"reduction dims differ: {K} vs {Kb}"
    return M, Nn, K


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _scale_desc(granularity, a_scale_inv, b_scale_inv, trans_a, trans_b, M, Nn, K):
    """-> (mode, sa_m, sa_k, sb_n, sb_k, sa_block, sb_block)"""
    if granularity == ScalingGranularity.TENSORWISE:
        _check(a_scale_inv.numel() == 1 and b_scale_inv.numel() == 1, "tensorwise scales must be scalars")
        return 0, 0, 0, 0, 0, 1, 1
    if granularity == ScalingGranularity.ROWWISE:
        _check(a_scale_inv.numel() == M, f"rowwise a_scale_inv must hold {M} values")
        _check(b_scale_inv.numel() == Nn, f"rowwise b_scale_inv must hold {Nn} values")
        return 0, 1, 0, 1, 0, 1, 1
    if granularity == ScalingGranularity.BLOCKWISE:
        kb = (K + 127) // 128
        if not trans_a and trans_b:  # NT: A [M,K] 1x128 scales [M,kb]; B [N,K] tile scales [N/128,kb]
            std = tuple(a_scale_inv.shape) == (M, kb) and tuple(b_scale_inv.shape) == ((Nn + 127) // 128, kb)
            if not std and tuple(a_scale_inv.shape) == (kb, M) and tuple(b_scale_inv.shape) == (kb, Nn):
                # both operands are transposed 128 x 1 column quantizations (K-contiguous data,
                # scales still [K/128, rows]): the wgrad product without a transposition pass
                return 1, 1, M, 1, Nn, 1, 1
            _check(tuple(a_scale_inv.shape) == (M, kb), "blockwise NT: a_scale_inv must be [M, K/128]")
            _check(tuple(b_scale_inv.shape) == ((Nn + 127) // 128, kb), "blockwise NT: b_scale_inv must be [N/128, K/128]")
            return 1, kb, 1, kb, 1, 1, 128
        if not trans_a and not trans_b:  # NN: B stored [K,N] with tile scales [K/128, N/128]
            nb = (Nn + 127) // 128
            _check(tuple(a_scale_inv.shape) == (M, kb), "blockwise NN: a_scale_inv must be [M, K/128]")
            _check(tuple(b_scale_inv.shape) == (kb, nb), "blockwise NN: b_scale_inv must be [K/128, N/128]")
            return 1, kb, 1, 1, nb, 1, 128
        if trans_a and not trans_b:  # TN: A stored [K,M] scales [K/128,M]; B stored [K,N] scales [K/128,N]
            _check(tuple(a_scale_inv.shape) == (kb, M), "blockwise TN: a_scale_inv must be [K/128, M]")
            _check(tuple(b_scale_inv.shape) == (kb, Nn), "blockwise TN: b_scale_inv must be [K/128, N]")
            return 1, 1, M, 1, Nn, 1, 1
        raise ValueError(f"Unsupported layout for blockwise FP8 GEMM: trans_a={trans_a}, trans_b={trans_b}")
    raise NotImplementedError(f"granularity {granularity} is handled by the MX GEMM entry points")


def launch_mx(a, a_scale, b, b_scale, out, trans_c, accumulate):
    """NT GEMM with E8M0 block scales on MX-quantized operands: ``a`` ``[M, K]`` and ``b`` ``[N, K]``
    codes (fp8, or ``float4_e2m1fn_x2`` with two codes per byte), scales ``[rows, K / 32]``."""
    N.require_cuda(a, b, a_scale, b_scale, out)
    fp4 = hasattr(torch, "float4_e2m1fn_x2") and a.dtype == torch.float4_e2m1fn_x2
    _check(a.dim() == 2 and b.dim() == 2, "MX GEMM expects 2-D operands")
    _check(a.dtype == b.dtype if fp4 else (a.dtype in _FP8 and b.dtype in _FP8), "operands must both be fp8 or both fp4")
    _check(out.dtype in _OUT, "out_dtype must be bfloat16, float16 or float32")
    a, b, a_scale, b_scale = a.contiguous(), b.contiguous(), a_scale.contiguous(), b_scale.contiguous()
    if trans_c:  # C^T = B . A^T
        a, b, a_scale, b_scale = b, a, b_scale, a_scale
    pack = 2 if fp4 else 1
    M, Nn = a.shape[0], b.shape[0]
    K = a.shape[1] * pack
    _check(b.shape[1] * pack == K, f"reduction dims differ: {K} vs {b.shape[1] * pack}")
    _check(K % 32 == 0, "K must be a multiple of 32")
    _check(a_scale.shape[0] == M and b_scale.shape[0] == Nn, "scale rows must match operand rows")
    _check(a_scale.shape[1] >= K // 32 and b_scale.shape[1] >= K // 32, "scales must hold K / 32 blocks per row")
    _check(a_scale.element_size() == 1 and b_scale.element_size() == 1, "scales must be E8M0 bytes")
    _check(tuple(out.shape) == (M, Nn) and out.is_contiguous(), f"out must be a contiguous {(M, Nn)} tensor")
    lib = N.lib()
    lda = ldb = K // pack
    ws = None
    ws_bytes = lib.pt_gemm_mx_workspace_bytes(M, Nn, K, lda, ldb, int(fp4))
    if ws_bytes:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device)
    N.check(
        lib.pt_gemm_mx(
            N.ptr(a), N.ptr(a_scale), N.ptr(b), N.ptr(b_scale), N.dtype_code(a.dtype),
            int(a.dtype == torch.float8_e5m2), int(b.dtype == torch.float8_e5m2),
            N.ptr(out), N.dtype_code(out.dtype), M, Nn, K, lda, ldb, a_scale.shape[1], b_scale.shape[1],
            int(accumulate), N.ptr(ws), ws_bytes, TILE_CFG, N.stream_of(a),
        )
    )
    return out


def _launch(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out, trans_c, granularity, accumulate):
    if granularity == ScalingGranularity.MX_BLOCKWISE:
        _check(not trans_a and trans_b, "MX_BLOCKWISE GEMM supports the NT layout only (trans_a=False, trans_b=True)")
        return launch_mx(a, a_scale_inv, b, b_scale_inv, out, trans_c, accumulate)
    N.require_cuda(a, b, a_scale_inv, b_scale_inv, out)
    _check(a.dtype in _FP8 and b.dtype in _FP8, "operands must be float8_e4m3fn / float8_e5m2")
    _check(out.dtype in _OUT, "out_dtype must be bfloat16, float16 or float32")
    _check(a_scale_inv.dtype == torch.float32 and b_scale_inv.dtype == torch.float32, "scales must be float32")
    a, b = a.contiguous(), b.contiguous()
    # per-row block scales of A may arrive as the [M, K/128] view of a block-major [K/128, M] tensor
    # (quant_fp8_blockwise_kmajor_impl(...)[1].t()): the kernel reads that layout in place
    a_kmajor = (granularity == ScalingGranularity.BLOCKWISE and not trans_a and a_scale_inv.dim() == 2
                and a_scale_inv.shape[1] > 1 and a_scale_inv.stride() == (1, a_scale_inv.shape[0]))
    if not a_kmajor:
        a_scale_inv = a_scale_inv.contiguous()
    b_scale_inv = b_scale_inv.contiguous()
    M, Nn, K = get_gemm_logical_shape(a, b, trans_a, trans_b)
    mode, sa_m, sa_k, sb_n, sb_k, sa_blk, sb_blk = _scale_desc(
        granularity, a_scale_inv, b_scale_inv, trans_a, trans_b, M, Nn, K
    )
    if a_kmajor and (sa_m, sa_k, sa_blk) == ((K + 127) // 128, 1, 1):
        sa_m, sa_k = 1, M
    elif a_kmajor:
        a_scale_inv = a_scale_inv.contiguous()
    if trans_c:
        # C^T = op(B)^T . op(A)^T: swap the operand roles, the kernel always writes row-major [M', N']
        a, b = b, a
        a_scale_inv, b_scale_inv = b_scale_inv, a_scale_inv
        trans_a, trans_b = (not trans_b), (not trans_a)
        M, Nn = Nn, M
        sa_m, sa_k, sb_n, sb_k = sb_n, sb_k, sa_m, sa_k
        sa_blk, sb_blk = sb_blk, sa_blk
    _check(tuple(out.shape) == (M, Nn) and out.is_contiguous(), f"out must be a contiguous {(M, Nn)} tensor")
    lib = N.lib()
    ws = None
    ws_bytes = lib.pt_gemm_fp8_workspace_bytes(M, Nn, K, int(trans_a), int(trans_b))
    if ws_bytes:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device)
    N.check(
        lib.pt_gemm_fp8(
            N.ptr(a), N.dtype_code(a.dtype), N.ptr(a_scale_inv),
            N.ptr(b), N.dtype_code(b.dtype), N.ptr(b_scale_inv),
            N.ptr(out), N.dtype_code(out.dtype), M, Nn, K, int(trans_a), int(trans_b),
            mode, sa_m, sa_k, sb_n, sb_k, sa_blk, sb_blk, int(accumulate),
            N.ptr(ws), ws_bytes, TILE_CFG, N.stream_of(a),
        )
    )
    return out


@torch.library.custom_op("primus_turbo::gemm_fp8_impl", mutates_args=(), device_types="cuda")
def gemm_fp8_impl(
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
) -> torch.Tensor:
    """``out = op(a) @ op(b)`` with the scaling of ``granularity`` (a ScalingGranularity value);
    ``trans_c`` returns the transposed product. ``default_backend`` is ignored (one backend)."""
    M, Nn, _ = get_gemm_logical_shape(a, b, trans_a, trans_b)
    shape = (Nn, M) if trans_c else (M, Nn)
    out = torch.empty(shape, dtype=out_dtype, device=a.device)
    return _launch(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out, trans_c, ScalingGranularity(granularity), False)


@gemm_fp8_impl.register_fake
def _gemm_fp8_impl_fake(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out_dtype, trans_c, granularity, default_backend):
    M, Nn, _ = get_gemm_logical_shape(a, b, trans_a, trans_b)
    if trans_c:
        M, Nn = Nn, M
    return torch.empty(M, Nn, dtype=out_dtype, device=a.device)


@torch.library.custom_op("primus_turbo::gemm_fp8_accum_impl", mutates_args={"out"}, device_types="cuda")
def gemm_fp8_accum_impl(
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
) -> None:
    """``out += op(a) @ op(b)``: the accumulation is folded into the GEMM epilogue (beta = 1)."""
    _launch(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out, trans_c, ScalingGranularity(granularity), True)


@gemm_fp8_accum_impl.register_fake
def _gemm_fp8_accum_impl_fake(a, a_scale_inv, trans_a, b, b_scale_inv, trans_b, out_dtype, trans_c, granularity, out, default_backend):
    M, Nn, _ = get_gemm_logical_shape(a, b, trans_a, trans_b)
    if trans_c:
        M, Nn = Nn, M
    assert tuple(out.shape) == (M, Nn), f"out shape {tuple(out.shape)} must equal {(M, Nn)}"
    return None
