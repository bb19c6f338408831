"""Grouped FP8 GEMM impl layer: the reference's ``grouped_gemm_fp8_impl`` /
``grouped_gemm_fp8_variable_k_impl`` / ``..._variable_k_accum_impl`` contracts
(primus_turbo/pytorch/kernels/grouped_gemm/grouped_gemm_fp8_impl.py:888-1022 of the reference)
on top of ``pt_grouped_gemm_fp8`` and ``pt_grouped_gemm_fp8_variable_k``.

One backend exists here, so ``default_backend``, ``num_cu`` and ``maybe_pre_sync`` are accepted
and ignored (the kernel is persistent over all CUs and never needs the group sizes on the
host). TENSORWISE / ROWWISE (vector scales applied in the epilogue), BLOCKWISE (fp32 scales per
128 block) and MX_BLOCKWISE (E8M0 bytes per 32 elements, MXFP8) are implemented.
"""

from __future__ import annotations

from typing import Optional

import torch

from primus_turbo import _native as N
from primus_turbo.pytorch.core.low_precision import ScalingGranularity

_FP8 = (torch.float8_e4m3fn, torch.float8_e5m2)

TILE_CFG = 0  # 0 = automatic; tests and the benchmark may pin 2 (256x128) or 3 (128x128)
MX_TILE_CFG = 0  # MX path: 0 = automatic, 1 = 256x256, 3 = 128x128, 4 = 256x256 with eight wavefronts (row groups only)


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _require_blockwise(granularity: int):
    if ScalingGranularity(granularity) != ScalingGranularity.BLOCKWISE:
        raise NotImplementedError(
            f"grouped FP8 GEMM: unknown granularity {ScalingGranularity(granularity)}"
        )


def _is_vec(granularity: int) -> bool:
    return ScalingGranularity(granularity) in (ScalingGranularity.TENSORWISE, ScalingGranularity.ROWWISE)


def _vec_stride(scale: torch.Tensor, n: int, what: str) -> int:
    """Stride (in floats) of a TENSORWISE (one element) or ROWWISE (``n`` elements) scale."""
    _check(scale.dtype == torch.float32, f"{what} must be float32")
    if scale.numel() == 1:
        return 0
    _check(scale.numel() == n, f"{what} must hold 1 or {n} elements, got {scale.numel()}")
    return 1


def _grouped_vec(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, out_dtype):
    """TENSORWISE / ROWWISE row groups: ``out[rows of g] = (a[rows of g] @ op(b[g])) * sa[m] * sb[g, n]``."""
    _check(not trans_a, "Only trans_a=False is supported.")
    N.require_cuda(a, b, a_scales, b_scales, group_offs)
    _check(a.dim() == 2 and b.dim() == 3, "a must be 2-D and b 3-D")
    _check(a.dtype in _FP8 and b.dtype in _FP8, "operands must be float8_e4m3fn / float8_e5m2")
    _check(out_dtype in (torch.float16, torch.bfloat16, torch.float32), "out_dtype must be float16, bfloat16 or float32")
    a, b = a.contiguous(), b.contiguous()
    a_scales, b_scales = a_scales.contiguous(), b_scales.contiguous()
    G = b.shape[0]
    M, K = a.shape
    Nn, Kb = (b.shape[1], b.shape[2]) if trans_b else (b.shape[2], b.shape[1])
    _check(K == Kb, f"reduction dims differ: {K} vs {Kb}")
    _check(group_offs.dtype == torch.int64 and group_offs.numel() == G + 1, "group_offs must be int64 [G + 1]")
    sa = _vec_stride(a_scales, M, "a_scales")
    sb = 0 if b_scales.numel() == 1 else 1
    _check(b_scales.dtype == torch.float32 and b_scales.numel() in (1, G * Nn), f"b_scales must hold 1 or G * N = {G * Nn} elements")
    out = torch.empty((M, Nn), dtype=out_dtype, device=a.device)
    lib = N.lib()
    ws_bytes = lib.pt_grouped_gemm_fp8_vec_workspace_bytes(G, M, Nn, K, int(trans_b))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes else None
    N.check(
        lib.pt_grouped_gemm_fp8_vec(
            N.ptr(a), N.dtype_code(a.dtype), N.ptr(a_scales), sa, N.ptr(b), N.dtype_code(b.dtype), N.ptr(b_scales), sb,
            Nn if sb else 0, N.ptr(out), N.dtype_code(out.dtype), N.ptr(group_offs.contiguous()), G, M, M, Nn, K,
            int(trans_b), N.ptr(ws), ws_bytes, _cfg_without_eight_waves(), N.stream_of(a),
        )
    )
    return out


def _variable_k_vec(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, accumulate):
    """TENSORWISE / ROWWISE variable K: ``out[g] = (a[rows of g]^T @ b[rows of g]) * sa[i] * sb[j]``
    over tightly packed groups (scales per column of ``a`` / ``b``, or scalars)."""
    _check(trans_a and not trans_b, "variable-K grouped GEMM computes a^T @ b (trans_a=True, trans_b=False)")
    N.require_cuda(a, b, a_scales, b_scales, group_offs, out)
    _check(a.dim() == 2 and b.dim() == 2 and a.shape[0] == b.shape[0], "a and b must be 2-D with the same row count")
    _check(a.dtype in _FP8 and b.dtype in _FP8, "operands must be float8_e4m3fn / float8_e5m2")
    a, b = a.contiguous(), b.contiguous()
    a_scales, b_scales = a_scales.contiguous(), b_scales.contiguous()
    M, Ml = a.shape
    Nr = b.shape[1]
    G = group_offs.numel() - 1
    sl, sr = _vec_stride(a_scales, Ml, "a_scales"), _vec_stride(b_scales, Nr, "b_scales")
    want = (G, Nr, Ml) if trans_c else (G, Ml, Nr)
    _check(tuple(out.shape) == want and out.is_contiguous(), f"out must be a contiguous {want} tensor")
    lib = N.lib()
    ws_bytes = lib.pt_grouped_gemm_fp8_vec_variable_k_workspace_bytes(G, M, Ml, Nr)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=a.device)
    N.check(
        lib.pt_grouped_gemm_fp8_vec_variable_k(
            N.ptr(a), N.dtype_code(a.dtype), N.ptr(a_scales), sl, N.ptr(b), N.dtype_code(b.dtype), N.ptr(b_scales), sr,
            N.ptr(out), N.dtype_code(out.dtype), N.ptr(group_offs.contiguous()), G, M, Ml, Nr, int(trans_c),
            int(accumulate), N.ptr(ws), ws_bytes, _cfg_without_eight_waves(), N.stream_of(a),
        )
    )
    return out


def _cfg_without_eight_waves() -> int:
    """The pinned MX tile configuration for the entry points that have no eight-wavefront tile."""
    return 0 if MX_TILE_CFG == 4 else MX_TILE_CFG


def _is_mx(granularity: int) -> bool:
    return ScalingGranularity(granularity) == ScalingGranularity.MX_BLOCKWISE


def _u8(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(torch.uint8)


_FP4X2 = getattr(torch, "float4_e2m1fn_x2", None)


def _mx_pitch(t: torch.Tensor, kbytes: int) -> torch.Tensor:
    """Rows of ``t`` (uint8, last dim = ``kbytes`` K bytes) at the pitch the kernel reads: whole
    128-byte slabs, at least four, zeros behind the data. No copy when it already is."""
    need = max(512, -(-kbytes // 128) * 128)
    return t if t.shape[-1] == need else torch.nn.functional.pad(t, (0, need - t.shape[-1]))


def _grouped_mx(a, b, a_scales, b_scales, group_offs, group_offs_out, trans_a, trans_b, out_dtype):
    """MX row groups: ``out[oo[g] : oo[g+1]] = a[o[g] : o[g] + len_g] @ b[g]^T`` with ``a`` in
    the (possibly per-group padded) row layout of the grouped quantizer and the output packed
    by ``group_offs_out`` (over-allocated to the rows of ``a``; the tail is zero). Operands are
    both MXFP8 or both packed MXFP4."""
    _check(not trans_a and trans_b, "MX grouped GEMM only supports trans_a=False, trans_b=True (NT layout).")
    N.require_cuda(a, b, a_scales, b_scales, group_offs)
    _check(a.dim() == 2 and b.dim() == 3, "a must be 2-D and b 3-D")
    fp4 = _FP4X2 is not None and a.dtype == _FP4X2
    if fp4:
        _check(b.dtype == _FP4X2, "operands must both be float4_e2m1fn_x2")
    else:
        _check(a.dtype in _FP8 and b.dtype in _FP8, "operands must be float8_e4m3fn / float8_e5m2")
    _check(out_dtype in (torch.float16, torch.bfloat16, torch.float32), "out_dtype must be float16, bfloat16 or float32")
    G, Nn, kb = b.shape  # kb: K bytes of a row
    rows = a.shape[0]
    _check(a.shape[1] == kb, f"reduction dims differ: {a.shape[1]} vs {kb}")
    K = kb * 2 if fp4 else kb
    # (any such K: rows shorter than four whole 128-byte slabs are copied once into zero-padded
    # rows, _mx_pitch below; the reference's operators pad K to 128 and have no lower limit,
    # csrc/pytorch/quantization/quantization.cpp:971-1100)
    _check(K % 32 == 0, "MX grouped GEMM needs K to be a multiple of 32")
    _check(group_offs.dtype == torch.int64 and group_offs.numel() == G + 1, "group_offs must be int64 [G + 1]")
    a_s, b_s = _u8(a_scales), _u8(b_scales)
    _check(a_s.dim() == 2 and a_s.shape[0] == rows and a_s.shape[1] >= K // 32, "a_scales must be [rows, K/32]")
    _check(b_s.dim() == 3 and tuple(b_s.shape[:2]) == (G, Nn) and b_s.shape[2] >= K // 32, "b_scales must be [G, N, K/32]")
    _check(a_s.shape[1] % 4 == 0 and b_s.shape[2] % 4 == 0, "scale rows must be multiples of 4 bytes")
    da, db = N.dtype_code(a.dtype), N.dtype_code(b.dtype)
    a, b = _mx_pitch(_u8(a), kb), _mx_pitch(_u8(b), kb)
    out = torch.empty((rows, Nn), dtype=out_dtype, device=a.device)
    oo = None if group_offs_out is None else group_offs_out.contiguous()
    # word-major scale copies pay once the K loop is long (measured: MXFP8 from K = 4096, MXFP4 from K = 2048)
    ws_bytes = N.lib().pt_grouped_gemm_mx_workspace_bytes(G, rows, Nn, K) if K >= (2048 if fp4 else 4096) else 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes else None
    N.check(
        N.lib().pt_grouped_gemm_mx(
            N.ptr(a), da, N.ptr(a_s), a.shape[1], a_s.shape[1], N.ptr(b), db, N.ptr(b_s), b.shape[2], b_s.shape[2], N.ptr(out),
            N.dtype_code(out.dtype), N.ptr(group_offs.contiguous()), N.ptr(oo), G, rows, rows, Nn, K, N.ptr(ws), ws_bytes,
            MX_TILE_CFG, N.stream_of(a),
        )
    )
    return out


def _variable_k_mx(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, accumulate):
    """MX variable K: ``out[g] = a[:, p[g]:p[g+1]] @ b[:, p[g]:p[g+1]]^T`` over the transposed
    column-direction outputs of the grouped quantizer (both K-contiguous already); ``p`` counts
    elements (multiples of 128, MXFP4 256)."""
    _check(not trans_a and not trans_b, "MX variable-K grouped GEMM takes both operands transposed already")
    N.require_cuda(a, b, a_scales, b_scales, group_offs, out)
    _check(a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[1], "a and b must be 2-D with the same padded length")
    fp4 = _FP4X2 is not None and a.dtype == _FP4X2
    if fp4:
        _check(b.dtype == _FP4X2, "operands must both be float4_e2m1fn_x2")
    else:
        _check(a.dtype in _FP8 and b.dtype in _FP8, "operands must be float8_e4m3fn / float8_e5m2")
    if trans_c:
        a, b, a_scales, b_scales = b, a, b_scales, a_scales
    Ml = a.shape[0]
    ld = a.shape[1] * (2 if fp4 else 1)
    Nr = b.shape[0]
    G = group_offs.numel() - 1
    _check(ld % (256 if fp4 else 128) == 0, "the padded length must be a multiple of 128 (MXFP4: 256)")
    a_s, b_s = _u8(a_scales), _u8(b_scales)
    _check(tuple(a_s.shape) == (Ml, ld // 32) and tuple(b_s.shape) == (Nr, ld // 32), "scales must be [rows, padded length / 32]")
    _check(tuple(out.shape) == (G, Ml, Nr) and out.is_contiguous(), f"out must be a contiguous {(G, Ml, Nr)} tensor")
    da, db = N.dtype_code(a.dtype), N.dtype_code(b.dtype)
    a, b = _u8(a), _u8(b)
    ws_bytes = N.lib().pt_grouped_gemm_mx_variable_k_workspace_bytes(Ml, Nr, ld) if ld >= 1024 else 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device) if ws_bytes else None
    N.check(
        N.lib().pt_grouped_gemm_mx_variable_k(
            N.ptr(a), da, N.ptr(a_s), N.ptr(b), db, N.ptr(b_s), N.ptr(out),
            N.dtype_code(out.dtype), N.ptr(group_offs.contiguous()), G, Ml, Nr, ld, int(accumulate), N.ptr(ws), ws_bytes,
            _cfg_without_eight_waves(), N.stream_of(a),
        )
    )
    return out


@torch.library.custom_op("primus_turbo::grouped_gemm_fp8_impl", mutates_args=(), device_types="cuda")
def grouped_gemm_fp8_impl(
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
    """``out[offs[g]:offs[g+1]] = a[offs[g]:offs[g+1]] @ op(b[g])``; rows past ``offs[G]`` are zero.

    ``a`` ``[M, K]`` fp8 with row scales stored ``[K/128, M]``; ``b`` ``[G, N, K]`` (``trans_b``)
    or ``[G, K, N]`` fp8 with 128 x 128 tile scales."""
    if _is_mx(granularity):
        return _grouped_mx(a, b, a_scales, b_scales, group_offs, group_offs_out, trans_a, trans_b, out_dtype)
    if _is_vec(granularity):
        _check(group_offs_out is None, "group_offs_out belongs to the MX grouped path")
        return _grouped_vec(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, out_dtype)
    _require_blockwise(granularity)
    _check(not trans_a, "Only trans_a=False is supported.")
    _check(group_offs_out is None, "group_offs_out belongs to the MX grouped path")
    N.require_cuda(a, b, a_scales, b_scales, group_offs)
    _check(a.dim() == 2 and b.dim() == 3, "a must be 2-D and b 3-D")
    _check(a.dtype in _FP8 and b.dtype in _FP8, "operands must be float8_e4m3fn / float8_e5m2")
    _check(out_dtype in (torch.float16, torch.bfloat16), "out_dtype must be float16 or bfloat16")
    _check(group_offs.dtype == torch.int64 and group_offs.numel() == b.shape[0] + 1, "group_offs must be int64 [G + 1]")
    a, b = a.contiguous(), b.contiguous()
    a_scales, b_scales = a_scales.contiguous(), b_scales.contiguous()
    G = b.shape[0]
    M, K = a.shape
    Nn, Kb = (b.shape[1], b.shape[2]) if trans_b else (b.shape[2], b.shape[1])
    _check(K == Kb, f"reduction dims differ: {K} vs {Kb}")
    kb, nb = (K + 127) // 128, (Nn + 127) // 128
    _check(tuple(a_scales.shape) == (kb, M), f"a_scales must be [K/128, M] = {(kb, M)}, got {tuple(a_scales.shape)}")
    want_b = (G, nb, kb) if trans_b else (G, kb, nb)
    _check(tuple(b_scales.shape) == want_b, f"b_scales must be {want_b}, got {tuple(b_scales.shape)}")
    out = torch.empty((M, Nn), dtype=out_dtype, device=a.device)
    lib = N.lib()
    ws = None
    ws_bytes = lib.pt_grouped_gemm_fp8_workspace_bytes(G, M, Nn, K, int(trans_b))
    if ws_bytes:
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a.device)
    N.check(
        lib.pt_grouped_gemm_fp8(
            N.ptr(a), N.dtype_code(a.dtype), N.ptr(a_scales),
            N.ptr(b), N.dtype_code(b.dtype), N.ptr(b_scales),
            N.ptr(out), N.dtype_code(out.dtype), N.ptr(group_offs), G, M, M, Nn, K, int(trans_b),
            N.ptr(ws), ws_bytes, TILE_CFG, N.stream_of(a),
        )
    )
    return out


@grouped_gemm_fp8_impl.register_fake
def _grouped_gemm_fp8_impl_fake(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b, out_dtype,
                                granularity, num_cu, default_backend, maybe_pre_sync=False, group_offs_out=None):
    assert a.dim() == 2 and b.dim() == 3
    n = b.shape[-2] if trans_b else b.shape[-1]
    return torch.empty((a.shape[0], n), device=a.device, dtype=out_dtype)


def _variable_k(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, accumulate):
    """``trans_a=True, trans_b=False``: ``a [Mp, Ml]``, ``b [Mp, Nr]`` (the reference's layout; both get
    transposed into a workspace). ``trans_a=False, trans_b=True``: ``a [Ml, Mp]``, ``b [Nr, Mp]`` with
    the padded rows contiguous already (``Mp % 128 == 0``): read in place."""
    kmajor = (not trans_a) and trans_b
    _check(kmajor or (trans_a and not trans_b),
           "variable-K grouped GEMM computes a^T @ b (trans_a=True, trans_b=False) or, with both operands "
           "transposed already, a @ b^T (trans_a=False, trans_b=True)")
    N.require_cuda(a, b, a_scales, b_scales, group_offs, out)
    r = 1 if kmajor else 0  # the axis of the (padded) rows
    _check(a.dim() == 2 and b.dim() == 2 and a.shape[r] == b.shape[r], "a and b must be 2-D with the same row count")
    _check(a.dtype in _FP8 and b.dtype in _FP8, "operands must be float8_e4m3fn / float8_e5m2")
    a, b = a.contiguous(), b.contiguous()
    a_scales, b_scales = a_scales.contiguous(), b_scales.contiguous()
    Mp, Ml, Nr = a.shape[r], a.shape[1 - r], b.shape[1 - r]
    G = group_offs.numel() - 1
    _check(not kmajor or Mp % 128 == 0, "K-major operands need a padded row count that is a multiple of 128")
    _check(a_scales.dim() == 2 and a_scales.shape[1] == Ml, "a_scales must be [rows/128, Ml]")
    _check(b_scales.dim() == 2 and b_scales.shape[1] == Nr, "b_scales must be [rows/128, Nr]")
    want = (G, Nr, Ml) if trans_c else (G, Ml, Nr)
    _check(tuple(out.shape) == want and out.is_contiguous(), f"out must be a contiguous {want} tensor")
    lib = N.lib()
    ws, ws_bytes = None, 0
    if not kmajor:
        ws_bytes = lib.pt_grouped_gemm_fp8_variable_k_workspace_bytes(Mp, Ml, Nr)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=a.device)
    N.check(
        lib.pt_grouped_gemm_fp8_variable_k(
            N.ptr(a), N.dtype_code(a.dtype), N.ptr(a_scales),
            N.ptr(b), N.dtype_code(b.dtype), N.ptr(b_scales),
            N.ptr(out), N.dtype_code(out.dtype), N.ptr(group_offs), G, Mp, Ml, Nr, int(trans_c), int(accumulate),
            int(kmajor), N.ptr(ws), ws_bytes, TILE_CFG, N.stream_of(a),
        )
    )
    return out


@torch.library.custom_op("primus_turbo::grouped_gemm_fp8_variable_k_impl", mutates_args=(), device_types="cuda")
def grouped_gemm_fp8_variable_k_impl(
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
    """``out[g] = a[p[g]:p[g+1]]^T @ b[p[g]:p[g+1]]`` (transposed when ``trans_c``) over the
    segment-padded column quantizations; ``group_offs`` holds the padded offsets ``p``."""
    G = group_offs.numel() - 1
    if _is_mx(granularity):
        shape = (G, b.shape[0], a.shape[0]) if trans_c else (G, a.shape[0], b.shape[0])
        out = torch.empty(shape, dtype=out_dtype, device=a.device)
        return _variable_k_mx(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, False)
    if _is_vec(granularity):
        shape = (G, b.shape[1], a.shape[1]) if trans_c else (G, a.shape[1], b.shape[1])
        out = torch.empty(shape, dtype=out_dtype, device=a.device)
        return _variable_k_vec(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, False)
    _require_blockwise(granularity)
    f = 0 if ((not trans_a) and trans_b) else 1  # the free axis: 0 when the operands come K-major
    shape = (G, b.shape[f], a.shape[f]) if trans_c else (G, a.shape[f], b.shape[f])
    out = torch.empty(shape, dtype=out_dtype, device=a.device)
    return _variable_k(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, False)


@grouped_gemm_fp8_variable_k_impl.register_fake
def _grouped_gemm_fp8_variable_k_impl_fake(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b,
                                           trans_c, out_dtype, granularity, num_cu, default_backend,
                                           maybe_pre_sync=False):
    G = group_offs.numel() - 1
    f = 0 if (_is_mx(granularity) or ((not trans_a) and trans_b and not _is_vec(granularity))) else 1
    shape = (G, b.shape[f], a.shape[f]) if trans_c else (G, a.shape[f], b.shape[f])
    return torch.empty(shape, dtype=out_dtype, device=a.device)


@torch.library.custom_op("primus_turbo::grouped_gemm_fp8_variable_k_accum_impl", mutates_args={"out"}, device_types="cuda")
def grouped_gemm_fp8_variable_k_accum_impl(
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
    """Same product, added into ``out`` in the GEMM epilogue (beta = 1)."""
    if _is_mx(granularity):
        _variable_k_mx(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, True)
        return
    if _is_vec(granularity):
        _variable_k_vec(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, True)
        return
    _require_blockwise(granularity)
    _variable_k(a, b, a_scales, b_scales, group_offs, trans_a, trans_b, trans_c, out, True)


@grouped_gemm_fp8_variable_k_accum_impl.register_fake
def _grouped_gemm_fp8_variable_k_accum_impl_fake(a, b, a_scales, b_scales, group_lens, group_offs, trans_a, trans_b,
                                                 trans_c, out_dtype, granularity, num_cu, default_backend, out,
                                                 maybe_pre_sync=False):
    return None
