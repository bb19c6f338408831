"""Quantizer impl layer: output allocation + shape rules + one C-ABI call per op.

Mirrors the split of the reference, where Python impls
(primus_turbo/pytorch/kernels/quantization/quantization_impl.py) call dispatcher ops
of the namespace ``primus_turbo_cpp_extension`` (csrc/pytorch/bindings_pytorch.cpp:34-93)
whose C++ bodies allocate outputs and launch kernels
(csrc/pytorch/quantization/quantization.cpp). Here the same op names are registered
from Python; their bodies allocate with torch and hand raw pointers to
libprimus_turbo_amd.so on the current stream.
"""

from __future__ import annotations

import os
from typing import List, Optional, Tuple

import torch

from primus_turbo import _native as N

_HP_DTYPES = (torch.bfloat16, torch.float16, torch.float32)
_FP8_DTYPES = (torch.float8_e4m3fn, torch.float8_e5m2)

_ext = torch.library.Library("primus_turbo_cpp_extension", "DEF")


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _check_fp8_out(dtype: torch.dtype) -> None:
    if dtype in (torch.float8_e4m3fnuz, torch.float8_e5m2fnuz):
        raise RuntimeError("FNUZ FP8 encodings are not produced on gfx950; use float8_e4m3fn / float8_e5m2")
    _check(dtype in _FP8_DTYPES, "dest_dtype must be float8_e4m3fn or float8_e5m2")


def _bmn(shape, axis: int) -> Tuple[int, int, int]:
    """View a tensor as [B, M, N] with M = the reduced axis
    (csrc/pytorch/quantization/quantization.cpp:92-108)."""
    if len(shape) == 0:
        return 1, 1, 1
    B = 1
    for s in shape[:axis]:
        B *= s
    Nn = 1
    for s in shape[axis + 1 :]:
        Nn *= s
    return B, shape[axis], Nn


# ---------------------------------------------------------------------------
# quantize_fp8_tensorwise(Tensor input, ScalarType dest_dtype, Tensor? scale_opt=None) -> Tensor[]
# ---------------------------------------------------------------------------
_ext.define("quantize_fp8_tensorwise(Tensor input, ScalarType dest_dtype, Tensor? scale_opt=None) -> Tensor[]")


# Which launch structure the dynamic tensorwise quantizer takes.
#   "fused"    one launch with a grid-wide amax exchange (x read once). Needs every workgroup of the
#              launch resident at once, which holds while nothing else keeps compute units busy
#              for long; the exchange words of eager calls live in the library's static scratch.
#   "two_pass" two launches, no exchange (x read twice): independent of what else runs on the GPU.
# Default: fused for eager calls, two_pass under HIP-graph capture (a replay may run beside any
# other work, and the static scratch is keyed by the capture stream, which every graph shares).
# PRIMUS_TURBO_TENSORWISE_MODE=fused|two_pass or set_tensorwise_mode() override both.
_TENSORWISE_MODES = ("auto", "fused", "two_pass")
_tensorwise_mode = os.environ.get("PRIMUS_TURBO_TENSORWISE_MODE", "auto")
if _tensorwise_mode not in _TENSORWISE_MODES:
    raise RuntimeError(f"PRIMUS_TURBO_TENSORWISE_MODE must be one of {_TENSORWISE_MODES}")


def set_tensorwise_mode(mode: str) -> str:
    """Select the launch structure of the dynamic tensorwise quantizer; returns the previous mode.
    Callers that run quantizers on several streams at once, or beside long kernels of other
    streams, want "two_pass"."""
    global _tensorwise_mode
    _check(mode in _TENSORWISE_MODES, f"mode must be one of {_TENSORWISE_MODES}")
    prev, _tensorwise_mode = _tensorwise_mode, mode
    return prev


def _quantize_fp8_tensorwise(input: torch.Tensor, dest_dtype: torch.dtype, scale_opt: Optional[torch.Tensor] = None):
    N.require_cuda(input, scale_opt)
    _check(input.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dest_dtype)
    _check(input.is_contiguous(), "input must be contiguous")
    lib = N.lib()
    out = torch.empty_like(input, dtype=dest_dtype)
    scale_inv = torch.empty((), dtype=torch.float32, device=input.device)
    scale_in = None
    if scale_opt is not None:
        _check(scale_opt.numel() == 1, "tensorwise scale must be scalar tensor")
        scale_in = scale_opt.to(torch.float32).contiguous()
    capturing = torch.cuda.is_current_stream_capturing()
    mode = _tensorwise_mode
    if mode == "auto":
        mode = "two_pass" if capturing else "fused"
    head = (N.ptr(input), N.dtype_code(input.dtype), input.numel(), N.ptr(out), N.dtype_code(dest_dtype))
    if scale_in is None and mode == "two_pass":
        # (the partial maxima need no zero-fill; the buffer comes from the capture's own pool)
        ws = torch.empty(lib.pt_quantize_fp8_tensorwise_workspace_bytes(), dtype=torch.uint8, device=input.device)
        N.check(lib.pt_quantize_fp8_tensorwise_two_pass(*head, N.ptr(scale_inv), N.ptr(ws), ws.numel(), N.stream_of(input)))
        return [out, scale_inv]
    if scale_in is not None:  # static scale: one cast launch, no exchange and no workspace
        N.check(lib.pt_quantize_fp8_tensorwise(*head, N.ptr(scale_in), N.ptr(scale_inv), None, 0, N.stream_of(input)))
        return [out, scale_inv]
    status = N.PT_ERR_WORKSPACE
    if not capturing:
        # The grid exchange of the fused kernel keeps its words in the library's static device
        # scratch (one slot set per stream handle): no per-call allocation or fill. A lost exchange
        # shows as NaN in scale_inv (see the header), so nothing is read back here.
        status = lib.pt_quantize_fp8_tensorwise_static(*head, None, N.ptr(scale_inv), None, N.stream_of(input))
    if status == N.PT_ERR_WORKSPACE:
        # under capture (every graph captured on torch's capture stream would share that stream's
        # static slot set, and replays of two graphs may overlap), or with more stream handles on
        # this device than the static scratch has slot sets: a zero-filled workspace of this call
        ws = N.zeroed_workspace(input.device, lib.pt_quantize_fp8_tensorwise_workspace_bytes())
        status = lib.pt_quantize_fp8_tensorwise(*head, None, N.ptr(scale_inv), N.ptr(ws), ws.numel(), N.stream_of(input))
    N.check(status)
    return [out, scale_inv]


def _quantize_fp8_tensorwise_meta(input, dest_dtype, scale_opt=None):
    return [
        torch.empty_like(input, dtype=dest_dtype),
        torch.empty((), dtype=torch.float32, device=input.device),
    ]


_ext.impl("quantize_fp8_tensorwise", _quantize_fp8_tensorwise, "CUDA")
_ext.impl("quantize_fp8_tensorwise", _quantize_fp8_tensorwise, "CPU")  # raises: no CPU path
_ext.impl("quantize_fp8_tensorwise", _quantize_fp8_tensorwise_meta, "Meta")

# ---------------------------------------------------------------------------
# dequantize_fp8_tensorwise(Tensor input, Tensor scale_inv, ScalarType dest_dtype) -> Tensor
# ---------------------------------------------------------------------------
_ext.define("dequantize_fp8_tensorwise(Tensor input, Tensor scale_inv, ScalarType dest_dtype) -> Tensor")


def _dequantize_fp8_tensorwise(input: torch.Tensor, scale_inv: torch.Tensor, dest_dtype: torch.dtype):
    N.require_cuda(input, scale_inv)
    _check(dest_dtype in _HP_DTYPES, "dest_dtype must be bfloat16, float16 or float32")
    _check(input.dtype in _FP8_DTYPES, "input must be float8_e4m3fn or float8_e5m2")
    _check(scale_inv.numel() == 1, "tensorwise scale_inv must be scalar tensor")
    _check(scale_inv.dtype == torch.float32, "scale_inv must be float32")
    x = input.contiguous()
    out = torch.empty_like(x, dtype=dest_dtype)
    N.check(
        N.lib().pt_dequantize_fp8_tensorwise(
            N.ptr(x), N.dtype_code(x.dtype), x.numel(), N.ptr(scale_inv), N.ptr(out), N.dtype_code(dest_dtype),
            N.stream_of(x),
        )
    )
    return out


def _dequantize_fp8_tensorwise_meta(input, scale_inv, dest_dtype):
    return torch.empty_like(input, dtype=dest_dtype)


_ext.impl("dequantize_fp8_tensorwise", _dequantize_fp8_tensorwise, "CUDA")
_ext.impl("dequantize_fp8_tensorwise", _dequantize_fp8_tensorwise, "CPU")
_ext.impl("dequantize_fp8_tensorwise", _dequantize_fp8_tensorwise_meta, "Meta")

# ---------------------------------------------------------------------------
# quantize_fp8_rowwise(Tensor input, ScalarType dest_dtype, int axis, Tensor? scale_opt=None) -> Tensor[]
# ---------------------------------------------------------------------------
_ext.define("quantize_fp8_rowwise(Tensor input, ScalarType dest_dtype, int axis, Tensor? scale_opt=None) -> Tensor[]")


def _valid_axis(axis: int, ndim: int) -> int:
    a = axis if axis >= 0 else ndim + axis
    _check(0 <= a < ndim, f"axis={axis} is out of range for a {ndim}-D tensor")
    return a


def _quantize_fp8_rowwise(input: torch.Tensor, dest_dtype: torch.dtype, axis: int, scale_opt=None):
    N.require_cuda(input, scale_opt)
    _check(input.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dest_dtype)
    _check(input.is_contiguous(), "input must be contiguous")
    a = _valid_axis(axis, input.dim())
    scale_shape = list(input.shape)
    scale_shape[a] = 1
    B, M, Nn = _bmn(list(input.shape), a)
    out = torch.empty_like(input, dtype=dest_dtype)
    scale_inv = torch.empty(scale_shape, dtype=torch.float32, device=input.device)
    scale_in = None
    if scale_opt is not None:
        _check(list(scale_opt.shape) == scale_shape, "scale shape must match input with size 1 along axis")
        scale_in = scale_opt.to(torch.float32).contiguous()
    N.check(
        N.lib().pt_quantize_fp8_rowwise(
            N.ptr(input), N.dtype_code(input.dtype), B, M, Nn, N.ptr(out), N.dtype_code(dest_dtype),
            N.ptr(scale_in), N.ptr(scale_inv), N.stream_of(input),
        )
    )
    return [out, scale_inv]


def _quantize_fp8_rowwise_meta(input, dest_dtype, axis, scale_opt=None):
    a = axis if axis >= 0 else input.dim() + axis
    scale_shape = list(input.shape)
    scale_shape[a] = 1
    return [
        torch.empty_like(input, dtype=dest_dtype),
        torch.empty(scale_shape, dtype=torch.float32, device=input.device),
    ]


_ext.impl("quantize_fp8_rowwise", _quantize_fp8_rowwise, "CUDA")
_ext.impl("quantize_fp8_rowwise", _quantize_fp8_rowwise, "CPU")
_ext.impl("quantize_fp8_rowwise", _quantize_fp8_rowwise_meta, "Meta")

# ---------------------------------------------------------------------------
# dequantize_fp8_rowwise(Tensor input, Tensor scale_inv, int axis, ScalarType dest_dtype) -> Tensor
# ---------------------------------------------------------------------------
_ext.define("dequantize_fp8_rowwise(Tensor input, Tensor scale_inv, int axis, ScalarType dest_dtype) -> Tensor")


def _dequantize_fp8_rowwise(input: torch.Tensor, scale_inv: torch.Tensor, axis: int, dest_dtype: torch.dtype):
    N.require_cuda(input, scale_inv)
    _check(dest_dtype in _HP_DTYPES, "dest_dtype must be bfloat16, float16 or float32")
    _check(input.dtype in _FP8_DTYPES, "input must be float8_e4m3fn or float8_e5m2")
    _check(scale_inv.dtype == torch.float32, "rowwise scale_inv must be float32 tensor")
    _check(input.is_contiguous(), "input must be contiguous")
    _check(scale_inv.is_contiguous(), "scale_inv must be contiguous")
    a = _valid_axis(axis, input.dim())
    expect = list(input.shape)
    expect[a] = 1
    _check(list(scale_inv.shape) == expect, "scale_inv shape must match input shape with size 1 along axis")
    B, M, Nn = _bmn(list(input.shape), a)
    out = torch.empty_like(input, dtype=dest_dtype)
    N.check(
        N.lib().pt_dequantize_fp8_rowwise(
            N.ptr(input), N.dtype_code(input.dtype), B, M, Nn, N.ptr(scale_inv), N.ptr(out),
            N.dtype_code(dest_dtype), N.stream_of(input),
        )
    )
    return out


def _dequantize_fp8_rowwise_meta(input, scale_inv, axis, dest_dtype):
    return torch.empty_like(input, dtype=dest_dtype)


_ext.impl("dequantize_fp8_rowwise", _dequantize_fp8_rowwise, "CUDA")
_ext.impl("dequantize_fp8_rowwise", _dequantize_fp8_rowwise, "CPU")
_ext.impl("dequantize_fp8_rowwise", _dequantize_fp8_rowwise_meta, "Meta")


# ===========================================================================
# Python impl entry points (same names as the reference's impl module)
# ===========================================================================
def quantize_fp8_tensorwise_impl(x: torch.Tensor, out_dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    x = x.contiguous()
    x_fp8, scale_inv = torch.ops.primus_turbo_cpp_extension.quantize_fp8_tensorwise(x, out_dtype, None)
    return x_fp8, scale_inv


def quantize_fp8_rowwise_impl(x: torch.Tensor, out_dtype: torch.dtype, axis: int):
    assert x.is_contiguous(), "The x tensor must be contiguous."
    x_fp8, scale_inv = torch.ops.primus_turbo_cpp_extension.quantize_fp8_rowwise(x, out_dtype, axis, None)
    return x_fp8, scale_inv


def dequantize_fp8_tensorwise_impl(x: torch.Tensor, out_dtype: torch.dtype, scale_inv: torch.Tensor):
    return torch.ops.primus_turbo_cpp_extension.dequantize_fp8_tensorwise(x, scale_inv, out_dtype)


def dequantize_fp8_rowwise_impl(x: torch.Tensor, out_dtype: torch.dtype, axis: int, scale_inv: torch.Tensor):
    assert x.is_contiguous(), "The x tensor must be contiguous."
    assert scale_inv.is_contiguous(), "The scale_inv tensor must be contiguous."
    return torch.ops.primus_turbo_cpp_extension.dequantize_fp8_rowwise(x, scale_inv, axis, out_dtype)


# ===========================================================================
# FP8 128-blockwise
# ===========================================================================
def ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def _need_block_128(block_size: int) -> None:
    _check(block_size == 128, f"only block_size=128 is built for the FP8 blockwise kernels, got {block_size}")


def _blockwise_launch(x, dtype, want_row: bool, want_col: bool):
    N.require_cuda(x)
    _check(x.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dtype)
    M, Nn = x.shape
    dev = x.device
    q_row = s_row = q_col = s_col = None
    if want_row:
        q_row = torch.empty((M, Nn), dtype=dtype, device=dev)
        s_row = torch.empty((M, ceil_div(Nn, 128)), dtype=torch.float32, device=dev)
    if want_col:
        q_col = torch.empty((M, Nn), dtype=dtype, device=dev)
        s_col = torch.empty((ceil_div(M, 128), Nn), dtype=torch.float32, device=dev)
    N.check(
        N.lib().pt_quantize_fp8_blockwise(
            N.ptr(x), N.dtype_code(x.dtype), M, Nn, N.dtype_code(dtype),
            N.ptr(q_row), N.ptr(s_row), N.ptr(q_col), N.ptr(s_col), N.stream_of(x),
        )
    )
    return q_row, s_row, q_col, s_col


@torch.library.custom_op("primus_turbo::quant_fp8_blockwise_impl", mutates_args=())
def quant_fp8_blockwise_impl(
    x: torch.Tensor, dtype: torch.dtype, axis: int, block_size: int = 128
) -> Tuple[torch.Tensor, torch.Tensor]:
    """1-D blockwise quantization of a contiguous 2-D tensor along ``axis``.

    axis 1 / -1: scales ``[M, cdiv(N, block)]``; axis 0 / -2: scales ``[cdiv(M, block), N]``.
    Returns ``(x_fp8, scale_inv)`` (the stored scale is 1/scale)."""
    assert x.is_contiguous() and x.dim() == 2, "Input must be 2D and contiguous"
    assert axis in (-2, -1, 0, 1), f"axis must be 0 or 1 (or -1, -2), got {axis}"
    _need_block_128(block_size)
    if axis % 2 == 1:
        q, s, _, _ = _blockwise_launch(x, dtype, True, False)
    else:
        _, _, q, s = _blockwise_launch(x, dtype, False, True)
    return q, s


@quant_fp8_blockwise_impl.register_fake
def _quant_fp8_blockwise_impl_fake(x, dtype, axis, block_size=128):
    assert x.dim() == 2, "Input must be 2D"
    assert axis in (-2, -1, 0, 1), f"axis must be 0 or 1 (or -1, -2), got {axis}"
    M, Nn = x.shape
    shape = (M, ceil_div(Nn, block_size)) if axis % 2 == 1 else (ceil_div(M, block_size), Nn)
    return (
        torch.empty((M, Nn), dtype=dtype, device=x.device),
        torch.empty(shape, dtype=torch.float32, device=x.device),
    )


@torch.library.custom_op("primus_turbo::quant_fp8_blockwise_dual_impl", mutates_args=())
def quant_fp8_blockwise_dual_impl(
    x: torch.Tensor, dtype: torch.dtype, block_size: int = 128
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Row (1 x block) and column (block x 1) quantization from one read of ``x``.

    Returns ``(x_fp8_row, scales_row [M, N/b], x_fp8_col, scales_col [M/b, N])``."""
    assert x.is_contiguous() and x.dim() == 2, "Input must be 2D and contiguous"
    _need_block_128(block_size)
    return _blockwise_launch(x, dtype, True, True)


@quant_fp8_blockwise_dual_impl.register_fake
def _quant_fp8_blockwise_dual_impl_fake(x, dtype, block_size=128):
    assert x.dim() == 2, "Input must be 2D"
    M, Nn = x.shape
    dev = x.device
    return (
        torch.empty((M, Nn), dtype=dtype, device=dev),
        torch.empty((M, ceil_div(Nn, block_size)), dtype=torch.float32, device=dev),
        torch.empty((M, Nn), dtype=dtype, device=dev),
        torch.empty((ceil_div(M, block_size), Nn), dtype=torch.float32, device=dev),
    )


@torch.library.custom_op("primus_turbo::quant_fp8_blockwise_dual_t_impl", mutates_args=())
def quant_fp8_blockwise_dual_t_impl(
    x: torch.Tensor, dtype: torch.dtype, block_size: int = 128
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """:func:`quant_fp8_blockwise_dual_impl` with the column codes emitted transposed and zero-padded:
    ``(x_fp8_row, scales_row [M, N/b], x_fp8_col_t [N, M_pad], scales_col [M/b, N])``, ``M_pad`` = ``M``
    rounded up to ``b`` -- the K-contiguous operand of the product that reduces over the rows of ``x``
    (wgrad). (No counterpart in the reference, whose GEMM backends read the untransposed layout.)"""
    N.require_cuda(x)
    _check(x.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dtype)
    _check(x.dim() == 2 and x.is_contiguous(), "Input must be 2D and contiguous")
    _need_block_128(block_size)
    M, Nn = x.shape
    Mp = ceil_div(M, block_size) * block_size
    dev = x.device
    q_row = torch.empty((M, Nn), dtype=dtype, device=dev)
    s_row = torch.empty((M, ceil_div(Nn, block_size)), dtype=torch.float32, device=dev)
    q_col_t = torch.empty((Nn, Mp), dtype=dtype, device=dev)
    s_col = torch.empty((ceil_div(M, block_size), Nn), dtype=torch.float32, device=dev)
    N.check(
        N.lib().pt_quantize_fp8_blockwise_t(
            N.ptr(x), N.dtype_code(x.dtype), M, Nn, N.dtype_code(dtype), N.ptr(q_row), N.ptr(s_row), None,
            N.ptr(q_col_t), Mp, N.ptr(s_col), N.stream_of(x),
        )
    )
    return q_row, s_row, q_col_t, s_col


@quant_fp8_blockwise_dual_t_impl.register_fake
def _quant_fp8_blockwise_dual_t_impl_fake(x, dtype, block_size=128):
    M, Nn = x.shape
    dev = x.device
    return (
        torch.empty((M, Nn), dtype=dtype, device=dev),
        torch.empty((M, ceil_div(Nn, block_size)), dtype=torch.float32, device=dev),
        torch.empty((Nn, ceil_div(M, block_size) * block_size), dtype=dtype, device=dev),
        torch.empty((ceil_div(M, block_size), Nn), dtype=torch.float32, device=dev),
    )


@torch.library.custom_op("primus_turbo::quant_fp8_blockwise_kmajor_impl", mutates_args=())
def quant_fp8_blockwise_kmajor_impl(
    x: torch.Tensor, dtype: torch.dtype, block_size: int, with_col_t: bool
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """The row direction of :func:`quant_fp8_blockwise_impl` with its scales stored block-major,
    ``scales_row_kmajor [N/b, M]`` (``.t()`` of it is the reference's ``[M, N/b]`` tensor, value for
    value): the layout the block-scaled GEMM reads, so no transposition pass precedes the product,
    and the quantizer writes whole cache lines of scales. ``with_col_t`` adds the transposed column
    codes and their scales as :func:`quant_fp8_blockwise_dual_t_impl` (empty tensors otherwise).
    ``(x_fp8_row, scales_row_kmajor, x_fp8_col_t, scales_col)``. (No counterpart in the reference.)"""
    N.require_cuda(x)
    _check(x.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dtype)
    _check(x.dim() == 2 and x.is_contiguous(), "Input must be 2D and contiguous")
    _need_block_128(block_size)
    M, Nn = x.shape
    Mp = ceil_div(M, block_size) * block_size
    dev = x.device
    q_row = torch.empty((M, Nn), dtype=dtype, device=dev)
    s_row = torch.empty((ceil_div(Nn, block_size), M), dtype=torch.float32, device=dev)
    q_col_t = torch.empty((Nn, Mp) if with_col_t else (0,), dtype=dtype, device=dev)
    s_col = torch.empty((ceil_div(M, block_size), Nn) if with_col_t else (0,), dtype=torch.float32, device=dev)
    N.check(
        N.lib().pt_quantize_fp8_blockwise_kmajor(
            N.ptr(x), N.dtype_code(x.dtype), M, Nn, N.dtype_code(dtype), N.ptr(q_row), N.ptr(s_row),
            N.ptr(q_col_t) if with_col_t else None, Mp if with_col_t else 0, N.ptr(s_col) if with_col_t else None,
            N.stream_of(x),
        )
    )
    return q_row, s_row, q_col_t, s_col


@quant_fp8_blockwise_kmajor_impl.register_fake
def _quant_fp8_blockwise_kmajor_impl_fake(x, dtype, block_size, with_col_t):
    M, Nn = x.shape
    dev = x.device
    return (
        torch.empty((M, Nn), dtype=dtype, device=dev),
        torch.empty((ceil_div(Nn, block_size), M), dtype=torch.float32, device=dev),
        torch.empty((Nn, ceil_div(M, block_size) * block_size) if with_col_t else (0,), dtype=dtype, device=dev),
        torch.empty((ceil_div(M, block_size), Nn) if with_col_t else (0,), dtype=torch.float32, device=dev),
    )


# quantize_fp8_blockwise_for_weight(Tensor input, ScalarType dest_dtype, int block_size) -> Tensor[]
_ext.define("quantize_fp8_blockwise_for_weight(Tensor input, ScalarType dest_dtype, int block_size) -> Tensor[]")


def _weight_shapes(w, block_size):
    if w.dim() == 2:
        B, (M, Nn) = 1, w.shape
        sshape = [ceil_div(M, block_size), ceil_div(Nn, block_size)]
    else:
        B, M, Nn = w.shape
        sshape = [B, ceil_div(M, block_size), ceil_div(Nn, block_size)]
    return B, M, Nn, sshape


def _quantize_fp8_blockwise_for_weight(input: torch.Tensor, dest_dtype: torch.dtype, block_size: int):
    N.require_cuda(input)
    _check(input.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dest_dtype)
    _check(input.dim() in (2, 3), "weight quant requires 2D or 3D input")
    _need_block_128(block_size)
    w = input.contiguous()
    B, M, Nn, sshape = _weight_shapes(w, block_size)
    q = torch.empty_like(w, dtype=dest_dtype)
    s = torch.empty(sshape, dtype=torch.float32, device=w.device)
    N.check(
        N.lib().pt_quantize_fp8_blockwise_weight(
            N.ptr(w), N.dtype_code(w.dtype), B, M, Nn, N.ptr(q), N.dtype_code(dest_dtype), N.ptr(s), N.stream_of(w)
        )
    )
    return [q, s]


def _quantize_fp8_blockwise_for_weight_meta(input, dest_dtype, block_size):
    _, _, _, sshape = _weight_shapes(input, block_size)
    return [
        torch.empty(input.shape, dtype=dest_dtype, device=input.device),
        torch.empty(sshape, dtype=torch.float32, device=input.device),
    ]


_ext.impl("quantize_fp8_blockwise_for_weight", _quantize_fp8_blockwise_for_weight, "CUDA")
_ext.impl("quantize_fp8_blockwise_for_weight", _quantize_fp8_blockwise_for_weight, "CPU")
_ext.impl("quantize_fp8_blockwise_for_weight", _quantize_fp8_blockwise_for_weight_meta, "Meta")


@torch.library.custom_op("primus_turbo::quant_fp8_blockwise_for_weight_impl", mutates_args=())
def quant_fp8_blockwise_for_weight_impl(
    w: torch.Tensor, dtype: torch.dtype, block_size: int = 128
) -> Tuple[torch.Tensor, torch.Tensor]:
    """One scale per block x block tile of a 2-D or 3-D weight -> ``(w_fp8, scale_inv)``."""
    assert w.dim() in (2, 3)
    q, s = torch.ops.primus_turbo_cpp_extension.quantize_fp8_blockwise_for_weight(w.contiguous(), dtype, block_size)
    return q, s


@quant_fp8_blockwise_for_weight_impl.register_fake
def _quant_fp8_blockwise_for_weight_impl_fake(w, dtype, block_size=128):
    assert w.dim() in (2, 3)
    q, s = _quantize_fp8_blockwise_for_weight_meta(w, dtype, block_size)
    return q, s


@torch.library.custom_op("primus_turbo::quant_fp8_blockwise_for_weight_dual_impl", mutates_args=())
def quant_fp8_blockwise_for_weight_dual_impl(
    w: torch.Tensor, dtype: torch.dtype, block_size: int = 128
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """:func:`quant_fp8_blockwise_for_weight_impl` plus, from the same read of ``w``, the codes
    transposed in their last two dimensions -> ``(w_fp8 [.., M, N], w_fp8_t [.., N, M], scale_inv)``.
    The transposed copy is the K-contiguous operand of the product that reduces over M (dgrad of a
    linear layer); it goes with ``scale_inv`` transposed in its last two dimensions. ``M % 16 == 0``.
    (No counterpart in the reference, whose GEMM backends read either layout.)"""
    N.require_cuda(w)
    _check(w.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dtype)
    _check(w.dim() in (2, 3), "weight quant requires 2D or 3D input")
    _need_block_128(block_size)
    w = w.contiguous()
    B, M, Nn, sshape = _weight_shapes(w, block_size)
    _check(M % 16 == 0, "the transposed copy needs a row count that is a multiple of 16")
    q = torch.empty_like(w, dtype=dtype)
    q_t = torch.empty(w.shape[:-2] + (Nn, M), dtype=dtype, device=w.device)
    sc = torch.empty(sshape, dtype=torch.float32, device=w.device)
    N.check(
        N.lib().pt_quantize_fp8_blockwise_weight_dual(
            N.ptr(w), N.dtype_code(w.dtype), B, M, Nn, N.ptr(q), N.ptr(q_t), M, N.dtype_code(dtype), N.ptr(sc),
            N.stream_of(w),
        )
    )
    return q, q_t, sc


@quant_fp8_blockwise_for_weight_dual_impl.register_fake
def _quant_fp8_blockwise_for_weight_dual_impl_fake(w, dtype, block_size=128):
    _, M, Nn, sshape = _weight_shapes(w, block_size)
    return (torch.empty(w.shape, dtype=dtype, device=w.device),
            torch.empty(w.shape[:-2] + (Nn, M), dtype=dtype, device=w.device),
            torch.empty(sshape, dtype=torch.float32, device=w.device))


def _dequant_block(q: torch.Tensor, scale_inv: torch.Tensor, out_dtype, B, M, Nn, bm, bn):
    N.require_cuda(q, scale_inv)
    _check(q.dtype in _FP8_DTYPES, "input must be float8_e4m3fn or float8_e5m2")
    _check(out_dtype in _HP_DTYPES, "out_dtype must be bfloat16, float16 or float32")
    _check(scale_inv.dtype == torch.float32, "scale_inv must be float32")
    s = scale_inv.contiguous()
    _check(s.numel() == B * ceil_div(M, bm) * ceil_div(Nn, bn), "scale_inv has the wrong number of elements")
    out = torch.empty(q.shape, dtype=out_dtype, device=q.device)
    N.check(
        N.lib().pt_dequantize_fp8_block(
            N.ptr(q), N.dtype_code(q.dtype), B, M, Nn, N.ptr(s), bm, bn, N.ptr(out), N.dtype_code(out_dtype),
            N.stream_of(q),
        )
    )
    return out


@torch.library.custom_op("primus_turbo::dequant_fp8_blockwise_impl", mutates_args=())
def dequant_fp8_blockwise_impl(
    x_fp8: torch.Tensor, scale_inv: torch.Tensor, out_dtype: torch.dtype, axis: int, block_size: int = 128
) -> torch.Tensor:
    """Inverse of :func:`quant_fp8_blockwise_impl` for the same ``axis``."""
    assert x_fp8.is_contiguous() and x_fp8.dim() == 2, "Input must be 2D and contiguous"
    assert axis in (-2, -1, 0, 1), f"axis must be 0 or 1 (or -1, -2), got {axis}"
    M, Nn = x_fp8.shape
    bm, bn = (1, block_size) if axis % 2 == 1 else (block_size, 1)
    return _dequant_block(x_fp8, scale_inv, out_dtype, 1, M, Nn, bm, bn)


@dequant_fp8_blockwise_impl.register_fake
def _dequant_fp8_blockwise_impl_fake(x_fp8, scale_inv, out_dtype, axis, block_size=128):
    assert x_fp8.dim() == 2, "Input must be 2D"
    return torch.empty(x_fp8.shape, dtype=out_dtype, device=x_fp8.device)


@torch.library.custom_op("primus_turbo::dequant_fp8_blockwise_for_weight_impl", mutates_args=())
def dequant_fp8_blockwise_for_weight_impl(
    w_fp8: torch.Tensor, scale_inv: torch.Tensor, out_dtype: torch.dtype, block_size: int = 128
) -> torch.Tensor:
    """Inverse of :func:`quant_fp8_blockwise_for_weight_impl` (2-D or 3-D)."""
    assert w_fp8.dim() in (2, 3)
    w = w_fp8.contiguous()
    B, M, Nn, _ = _weight_shapes(w, block_size)
    return _dequant_block(w, scale_inv, out_dtype, B, M, Nn, block_size, block_size)


@dequant_fp8_blockwise_for_weight_impl.register_fake
def _dequant_fp8_blockwise_for_weight_impl_fake(w_fp8, scale_inv, out_dtype, block_size=128):
    assert w_fp8.dim() in (2, 3)
    return torch.empty(w_fp8.shape, dtype=out_dtype, device=w_fp8.device)


# ---------------------------------------------------------------------------
# group offsets and the fused grouped row + segment-padded column quantizer
# ---------------------------------------------------------------------------
_ext.define("grouped_gemm_compute_offs(Tensor group_lens) -> Tensor")


def _group_offs(group_lens: torch.Tensor, align: int, want_padded_lens: bool):
    N.require_cuda(group_lens)
    _check(group_lens.dtype == torch.int64 and group_lens.dim() == 1, "group_lens must be a 1-D int64 tensor")
    gl = group_lens.contiguous()
    G = gl.numel()
    offs = torch.empty(G + 1, dtype=torch.int64, device=gl.device)
    padded = torch.empty(G, dtype=torch.int64, device=gl.device) if want_padded_lens else None
    N.check(N.lib().pt_compute_group_offs(N.ptr(gl), G, align, N.ptr(padded), N.ptr(offs), N.stream_of(gl)))
    return padded, offs


def _grouped_gemm_compute_offs(group_lens: torch.Tensor) -> torch.Tensor:
    return _group_offs(group_lens, 1, False)[1]


def _grouped_gemm_compute_offs_meta(group_lens):
    return torch.empty(group_lens.numel() + 1, dtype=torch.int64, device=group_lens.device)


_ext.impl("grouped_gemm_compute_offs", _grouped_gemm_compute_offs, "CUDA")
_ext.impl("grouped_gemm_compute_offs", _grouped_gemm_compute_offs, "CPU")
_ext.impl("grouped_gemm_compute_offs", _grouped_gemm_compute_offs_meta, "Meta")

_ext.define(
    "quantize_fp8_blockwise_segment_m_row_col(Tensor input, ScalarType dest_dtype, int block_size, "
    "Tensor group_lens, Tensor group_offs) -> Tensor[]"
)


def _segment_shapes(M, Nn, G, block_size):
    Mp = M + G * block_size
    return Mp, (ceil_div(Nn, block_size), M), (ceil_div(Mp, block_size), Nn)


def _quantize_fp8_blockwise_segment_m_row_col(input, dest_dtype, block_size, group_lens, group_offs):
    N.require_cuda(input, group_lens, group_offs)
    _check(input.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dest_dtype)
    _check(input.dim() == 2, "input must be 2D")
    _need_block_128(block_size)
    for t in (group_lens, group_offs):
        _check(t.dtype == torch.int64, "group_lens / group_offs must be int64")
        _check(t.is_contiguous(), "group_lens / group_offs must be contiguous")
    G = group_lens.numel()
    _check(group_offs.numel() == G + 1, "group_offs must have one more element than group_lens")
    x = input.contiguous()
    M, Nn = x.shape
    Mp, rs_shape, cs_shape = _segment_shapes(M, Nn, G, block_size)
    dev = x.device
    padded_lens, padded_offs = _group_offs(group_lens, block_size, True)
    q_row = torch.empty((M, Nn), dtype=dest_dtype, device=dev)
    q_col = torch.empty((Mp, Nn), dtype=dest_dtype, device=dev)
    s_row = torch.empty(rs_shape, dtype=torch.float32, device=dev)
    s_col = torch.empty(cs_shape, dtype=torch.float32, device=dev)
    N.check(
        N.lib().pt_quantize_fp8_blockwise_segment_m_row_col(
            N.ptr(x), N.dtype_code(x.dtype), M, Nn, N.dtype_code(dest_dtype), N.ptr(group_offs), N.ptr(padded_offs),
            G, N.ptr(q_row), N.ptr(s_row), N.ptr(q_col), N.ptr(s_col), N.stream_of(x),
        )
    )
    return [q_row, q_col, s_row, s_col, padded_lens, padded_offs]


def _quantize_fp8_blockwise_segment_m_row_col_meta(input, dest_dtype, block_size, group_lens, group_offs):
    M, Nn = input.shape
    G = group_lens.numel()
    Mp, rs_shape, cs_shape = _segment_shapes(M, Nn, G, block_size)
    dev = input.device
    return [
        torch.empty((M, Nn), dtype=dest_dtype, device=dev),
        torch.empty((Mp, Nn), dtype=dest_dtype, device=dev),
        torch.empty(rs_shape, dtype=torch.float32, device=dev),
        torch.empty(cs_shape, dtype=torch.float32, device=dev),
        torch.empty(G, dtype=torch.int64, device=dev),
        torch.empty(G + 1, dtype=torch.int64, device=dev),
    ]


_ext.impl("quantize_fp8_blockwise_segment_m_row_col", _quantize_fp8_blockwise_segment_m_row_col, "CUDA")
_ext.impl("quantize_fp8_blockwise_segment_m_row_col", _quantize_fp8_blockwise_segment_m_row_col, "CPU")
_ext.impl("quantize_fp8_blockwise_segment_m_row_col", _quantize_fp8_blockwise_segment_m_row_col_meta, "Meta")


@torch.library.custom_op("primus_turbo::quant_fp8_blockwise_segment_m_row_col_impl", mutates_args=())
def quant_fp8_blockwise_segment_m_row_col_impl(
    x: torch.Tensor,
    dtype: torch.dtype,
    block_size: int,
    group_lens: torch.Tensor,
    group_offs: torch.Tensor,
    gemm_other_dim: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Fused grouped quantizer: one read of the packed-M activation ``x [M, N]`` yields the
    row-quantized tensor (fwd / dgrad operand, scales stored ``[N/b, M]``) and the
    segment-padded column-quantized tensor (variable-K wgrad operand).

    Returns ``(x_fp8_row [M,N], x_fp8_col_padded [M+G*b,N], scales_row [N/b,M],
    scales_col_padded [(M+G*b)/b,N], padded_group_lens [G], padded_group_offs [G+1])``.
    ``gemm_other_dim`` is accepted for signature parity; there is a single kernel here."""
    assert x.is_contiguous() and x.dim() == 2
    r = torch.ops.primus_turbo_cpp_extension.quantize_fp8_blockwise_segment_m_row_col(
        x, dtype, block_size, group_lens, group_offs
    )
    return r[0], r[1], r[2], r[3], r[4], r[5]


@quant_fp8_blockwise_segment_m_row_col_impl.register_fake
def _quant_fp8_blockwise_segment_m_row_col_impl_fake(x, dtype, block_size, group_lens, group_offs, gemm_other_dim=None):
    r = _quantize_fp8_blockwise_segment_m_row_col_meta(x, dtype, block_size, group_lens, group_offs)
    return r[0], r[1], r[2], r[3], r[4], r[5]


def _segment_t_pitch(M: int, G: int, block_size: int) -> int:
    return ceil_div(M + G * block_size, block_size) * block_size


@torch.library.custom_op("primus_turbo::quant_fp8_blockwise_segment_m_row_col_t_impl", mutates_args=())
def quant_fp8_blockwise_segment_m_row_col_t_impl(
    x: torch.Tensor, dtype: torch.dtype, block_size: int, group_lens: torch.Tensor, group_offs: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """:func:`quant_fp8_blockwise_segment_m_row_col_impl` with the segment-padded column codes
    emitted transposed: ``x_fp8_col_t [N, Mp]`` (``Mp`` = ``M + G * b`` rounded up to ``b``), the
    K-contiguous operand of the variable-K wgrad product; everything else (row codes, both scale
    tensors, padded lens / offs) as there. (No counterpart in the reference, whose GEMM backends
    read the untransposed layout.)"""
    N.require_cuda(x, group_lens, group_offs)
    _check(x.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dtype)
    _check(x.dim() == 2 and x.is_contiguous(), "input must be 2D and contiguous")
    _need_block_128(block_size)
    for t in (group_lens, group_offs):
        _check(t.dtype == torch.int64 and t.is_contiguous(), "group_lens / group_offs must be contiguous int64")
    G = group_lens.numel()
    _check(group_offs.numel() == G + 1, "group_offs must have one more element than group_lens")
    M, Nn = x.shape
    _, rs_shape, cs_shape = _segment_shapes(M, Nn, G, block_size)
    ldt = _segment_t_pitch(M, G, block_size)
    dev = x.device
    padded_lens, padded_offs = _group_offs(group_lens, block_size, True)
    q_row = torch.empty((M, Nn), dtype=dtype, device=dev)
    q_col_t = torch.empty((Nn, ldt), dtype=dtype, device=dev)
    s_row = torch.empty(rs_shape, dtype=torch.float32, device=dev)
    s_col = torch.empty(cs_shape, dtype=torch.float32, device=dev)
    N.check(
        N.lib().pt_quantize_fp8_blockwise_segment_m_row_col_t(
            N.ptr(x), N.dtype_code(x.dtype), M, Nn, N.dtype_code(dtype), N.ptr(group_offs), N.ptr(padded_offs), G,
            N.ptr(q_row), N.ptr(s_row), None, N.ptr(q_col_t), ldt, N.ptr(s_col), N.stream_of(x),
        )
    )
    return q_row, q_col_t, s_row, s_col, padded_lens, padded_offs


@quant_fp8_blockwise_segment_m_row_col_t_impl.register_fake
def _quant_fp8_blockwise_segment_m_row_col_t_impl_fake(x, dtype, block_size, group_lens, group_offs):
    M, Nn = x.shape
    G = group_lens.numel()
    _, rs_shape, cs_shape = _segment_shapes(M, Nn, G, block_size)
    dev = x.device
    return (torch.empty((M, Nn), dtype=dtype, device=dev),
            torch.empty((Nn, _segment_t_pitch(M, G, block_size)), dtype=dtype, device=dev),
            torch.empty(rs_shape, dtype=torch.float32, device=dev), torch.empty(cs_shape, dtype=torch.float32, device=dev),
            torch.empty(G, dtype=torch.int64, device=dev), torch.empty(G + 1, dtype=torch.int64, device=dev))


_GLU_ACT = {"silu": 0, "gelu": 1}


@torch.library.custom_op("primus_turbo::glu_quant_fp8_blockwise_segment_m_row_col_impl", mutates_args=())
def glu_quant_fp8_blockwise_segment_m_row_col_impl(
    x: torch.Tensor, probs: torch.Tensor, row_mask: Optional[torch.Tensor], act: str, dtype: torch.dtype,
    block_size: int, group_lens: torch.Tensor, group_offs: torch.Tensor, transposed_col: bool,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Gated activation fused into the grouped quantizer: ``x [M, 2 N]`` is the fc1 output of an MoE
    expert MLP and the tensor quantized is ``y = T(act(x[:, :N]) * x[:, N:] * probs[:, None])`` (zero
    rows where ``row_mask`` is 0), i.e. what ``swiglu_with_probs`` / ``geglu_with_probs`` would store,
    which never travels through HBM here. Outputs as :func:`quant_fp8_blockwise_segment_m_row_col_impl`
    (``transposed_col=False``) or :func:`quant_fp8_blockwise_segment_m_row_col_t_impl` (``True``), bit
    for bit what those give on the stored activation. (No counterpart in the reference.)"""
    N.require_cuda(x, probs, row_mask, group_lens, group_offs)
    _check(act in _GLU_ACT, "act must be 'silu' or 'gelu'")
    _check(x.dtype in (torch.bfloat16, torch.float16), "input must be bfloat16 or float16")
    _check_fp8_out(dtype)
    _check(x.dim() == 2 and x.is_contiguous() and x.shape[1] % 2 == 0, "input must be a contiguous [M, 2 N] tensor")
    _need_block_128(block_size)
    M, Nn = x.shape[0], x.shape[1] // 2
    _check(probs.numel() == M, "probs must hold one value per row")
    p32 = probs.reshape(-1).to(torch.float32).contiguous()
    mask = None
    if row_mask is not None:
        _check(row_mask.numel() == M, "row_mask must hold one value per row")
        mask = row_mask.reshape(-1).to(torch.int64).contiguous()
    for t in (group_lens, group_offs):
        _check(t.dtype == torch.int64 and t.is_contiguous(), "group_lens / group_offs must be contiguous int64")
    G = group_lens.numel()
    _check(group_offs.numel() == G + 1, "group_offs must have one more element than group_lens")
    Mp, rs_shape, cs_shape = _segment_shapes(M, Nn, G, block_size)
    ldt = _segment_t_pitch(M, G, block_size)
    dev = x.device
    padded_lens, padded_offs = _group_offs(group_lens, block_size, True)
    q_row = torch.empty((M, Nn), dtype=dtype, device=dev)
    q_col = torch.empty((Nn, ldt) if transposed_col else (Mp, Nn), dtype=dtype, device=dev)
    s_row = torch.empty(rs_shape, dtype=torch.float32, device=dev)
    s_col = torch.empty(cs_shape, dtype=torch.float32, device=dev)
    N.check(
        N.lib().pt_glu_quantize_fp8_blockwise_segment_m_row_col(
            N.ptr(x), N.dtype_code(x.dtype), N.ptr(p32), N.ptr(mask), _GLU_ACT[act], M, Nn, N.dtype_code(dtype),
            N.ptr(group_offs), N.ptr(padded_offs), G, N.ptr(q_row), N.ptr(s_row),
            None if transposed_col else N.ptr(q_col), N.ptr(q_col) if transposed_col else None, ldt, N.ptr(s_col),
            N.stream_of(x),
        )
    )
    return q_row, q_col, s_row, s_col, padded_lens, padded_offs


@glu_quant_fp8_blockwise_segment_m_row_col_impl.register_fake
def _glu_quant_fp8_blockwise_segment_m_row_col_impl_fake(x, probs, row_mask, act, dtype, block_size, group_lens, group_offs,
                                                         transposed_col):
    M, Nn = x.shape[0], x.shape[1] // 2
    G = group_lens.numel()
    Mp, rs_shape, cs_shape = _segment_shapes(M, Nn, G, block_size)
    dev = x.device
    return (torch.empty((M, Nn), dtype=dtype, device=dev),
            torch.empty((Nn, _segment_t_pitch(M, G, block_size)) if transposed_col else (Mp, Nn), dtype=dtype, device=dev),
            torch.empty(rs_shape, dtype=torch.float32, device=dev), torch.empty(cs_shape, dtype=torch.float32, device=dev),
            torch.empty(G, dtype=torch.int64, device=dev), torch.empty(G + 1, dtype=torch.int64, device=dev))


# ---------------------------------------------------------------------------------------
# MX quantizers (E8M0 scale per 32 elements): MXFP8 and MXFP4
# reference: primus_turbo/pytorch/kernels/quantization/quantization_impl.py:496-569,814-835,
#            868-1010; shapes from csrc/pytorch/quantization/quantization.cpp:511-969
# ---------------------------------------------------------------------------------------
_MX_PAD = 128
_E8M0 = getattr(torch, "float8_e8m0fnu", torch.uint8)
_FP4X2 = getattr(torch, "float4_e2m1fn_x2", None)


# ---------------------------------------------------------------------------
# Pre-shuffled MX layouts: shuffle_scale(Tensor scale, int[] layout) -> Tensor and
# shuffle_weight(Tensor weight, int[] layout) -> Tensor of the reference
# (csrc/pytorch/bindings_pytorch.cpp, csrc/pytorch/shuffle/shuffle.cpp:15-83), their inverses, and the
# quantizers' shuffle_scale / shuffle_out outputs (csrc/pytorch/quantization/quantization.cpp:553-603).
# ---------------------------------------------------------------------------
_SHUFFLE_ROWS, _SHUFFLE_SCALE_M_ALIGN, _SHUFFLE_SCALE_N_ALIGN = 16, 256, 8


def _check_layout(layout):
    _check(len(layout) == 2, "layout must have exactly 2 elements")
    _check(tuple(layout) == (16, 16), "Unsupported shuffle layout.")


def _scale_pad(M: int, Nn: int) -> Tuple[int, int]:
    a, b = _SHUFFLE_SCALE_M_ALIGN, _SHUFFLE_SCALE_N_ALIGN
    return -(-M // a) * a, -(-Nn // b) * b


def _shuffle_scale_launch(scale: torch.Tensor, batch: int, M: int, Nn: int) -> torch.Tensor:
    """``batch`` stacked ``[M, Nn]`` E8M0 matrices -> ``[batch * M_pad, N_pad]`` shuffled."""
    Mp, Np = _scale_pad(M, Nn)
    out = torch.empty((batch * Mp, Np), dtype=torch.uint8, device=scale.device)
    N.check(N.lib().pt_shuffle_e8m0_scale(N.ptr(scale), N.ptr(out), batch, M, Nn, Mp, Np, 0, N.stream_of(scale)))
    return out.view(_E8M0)


_ext.define("shuffle_scale(Tensor scale, int[] layout) -> Tensor")


def _shuffle_scale(scale: torch.Tensor, layout: List[int]) -> torch.Tensor:
    N.require_cuda(scale)
    _check(scale.dtype == _E8M0, "Scale must be Float8_e8m0fnu.")
    _check(scale.dim() == 2, "Scale must be 2D")
    _check_layout(layout)
    return _shuffle_scale_launch(scale.contiguous(), 1, scale.shape[0], scale.shape[1])


def _shuffle_scale_meta(scale, layout):
    Mp, Np = _scale_pad(scale.shape[0], scale.shape[1])
    return torch.empty((Mp, Np), dtype=torch.uint8, device=scale.device).view(_E8M0)


_ext.impl("shuffle_scale", _shuffle_scale, "CUDA")
_ext.impl("shuffle_scale", _shuffle_scale, "CPU")  # raises: no CPU path
_ext.impl("shuffle_scale", _shuffle_scale_meta, "Meta")

_ext.define("unshuffle_scale(Tensor shuffled, int M, int N) -> Tensor")


def _unshuffle_scale(shuffled: torch.Tensor, M: int, Nn: int) -> torch.Tensor:
    """Inverse of ``shuffle_scale``: the plain ``[M, N]`` scales of a shuffled ``[M_pad, N_pad]`` tensor
    (no counterpart in the reference, whose GEMM backends read the shuffled form)."""
    N.require_cuda(shuffled)
    _check(shuffled.dtype == _E8M0 and shuffled.dim() == 2, "shuffled scale must be a 2-D Float8_e8m0fnu tensor")
    _check(tuple(shuffled.shape) == _scale_pad(M, Nn), f"shuffled scale of [{M}, {Nn}] must be {_scale_pad(M, Nn)}")
    shuffled = shuffled.contiguous()
    out = torch.empty((M, Nn), dtype=torch.uint8, device=shuffled.device)
    N.check(N.lib().pt_shuffle_e8m0_scale(N.ptr(shuffled), N.ptr(out), 1, M, Nn, shuffled.shape[0], shuffled.shape[1], 1,
                                          N.stream_of(shuffled)))
    return out.view(_E8M0)


_ext.impl("unshuffle_scale", _unshuffle_scale, "CUDA")
_ext.impl("unshuffle_scale", _unshuffle_scale, "CPU")
_ext.impl("unshuffle_scale", lambda s, M, Nn: torch.empty((M, Nn), dtype=torch.uint8, device=s.device).view(_E8M0), "Meta")


def _shuffle_codes_launch(codes: torch.Tensor, inverse: bool) -> torch.Tensor:
    rows, row_bytes = codes.numel() // codes.shape[-1], codes.shape[-1] * codes.element_size()
    out = torch.empty_like(codes)
    N.check(N.lib().pt_shuffle_mx_codes(N.ptr(codes), N.ptr(out), rows, row_bytes, int(inverse), N.stream_of(codes)))
    return out


def _check_weight(weight, layout):
    N.require_cuda(weight)
    _check(_FP4X2 is not None and weight.dtype == _FP4X2, "Weight must be Float4_e2m1fn_x2.")
    _check(weight.dim() == 2, "Weight must be 2D")
    _check(weight.is_contiguous(), "Weight must be contiguous")
    M, Nn = weight.shape
    _check(M % 16 == 0, f"M must be divisible by 16 for shuffled FP4. But got M={M}")
    _check(Nn % 32 == 0, f"N must be divisible by 32 for shuffled FP4. But got N={Nn}")
    _check_layout(layout)


_ext.define("shuffle_weight(Tensor weight, int[] layout) -> Tensor")
_ext.define("unshuffle_weight(Tensor shuffled, int[] layout) -> Tensor")


def _shuffle_weight(weight: torch.Tensor, layout: List[int]) -> torch.Tensor:
    _check_weight(weight, layout)
    return _shuffle_codes_launch(weight, False)


def _unshuffle_weight(shuffled: torch.Tensor, layout: List[int]) -> torch.Tensor:
    """Inverse of ``shuffle_weight`` (no counterpart in the reference)."""
    _check_weight(shuffled, layout)
    return _shuffle_codes_launch(shuffled, True)


for _name, _fn in (("shuffle_weight", _shuffle_weight), ("unshuffle_weight", _unshuffle_weight)):
    _ext.impl(_name, _fn, "CUDA")
    _ext.impl(_name, _fn, "CPU")
    _ext.impl(_name, lambda w, layout: torch.empty_like(w), "Meta")


def _apply_mx_shuffles(q, s, recipe, direction: str):
    """The ``shuffle_out`` / ``shuffle_scale`` forms of one direction's outputs ``q [.., R, W]`` /
    ``s [.., R, W / 32]``: a pass over the plain outputs of the quantizer. Batched scales are shuffled
    per matrix, each padded on its own (quantization.cpp:563-603)."""
    if q is None:
        return q, s
    if recipe.shuffle_out:
        R = q.shape[-2]
        what = "M" if direction == "rowwise" else "N"
        _check(R % _SHUFFLE_ROWS == 0,
               f"{what} must be divisible by {_SHUFFLE_ROWS} for shuffled {direction} output. But got {what}={R}")
        q = _shuffle_codes_op(q, False)
    if recipe.shuffle_scale:
        s = torch.ops.primus_turbo_cpp_extension.shuffle_scale_batched(s)
    return q, s


_ext.define("shuffle_scale_batched(Tensor scale) -> Tensor")


def _shuffle_scale_batched(scale: torch.Tensor) -> torch.Tensor:
    N.require_cuda(scale)
    batch = scale.shape[0] if scale.dim() == 3 else 1
    out = _shuffle_scale_launch(scale.contiguous(), batch, scale.shape[-2], scale.shape[-1])
    return out.view(batch, -1, out.shape[-1]) if scale.dim() == 3 else out


def _shuffle_scale_batched_meta(scale):
    Mp, Np = _scale_pad(scale.shape[-2], scale.shape[-1])
    return torch.empty(tuple(scale.shape[:-2]) + (Mp, Np), dtype=torch.uint8, device=scale.device).view(_E8M0)


_ext.impl("shuffle_scale_batched", _shuffle_scale_batched, "CUDA")
_ext.impl("shuffle_scale_batched", _shuffle_scale_batched_meta, "Meta")


def mx_plain_layout(q: torch.Tensor, scale: torch.Tensor, shuffled_out: bool, shuffled_scale: bool):
    """``(codes, scales)`` of a 2-D MX operand in the plain row-major layout that the GEMM and
    de-quantization kernels read, from outputs produced with ``shuffle_out`` / ``shuffle_scale``."""
    if shuffled_out:
        q = _shuffle_codes_op(q, True)
    if shuffled_scale:
        cols = q.shape[-1] * (2 if (_FP4X2 is not None and q.dtype == _FP4X2) else 1) // 32
        scale = torch.ops.primus_turbo_cpp_extension.unshuffle_scale(scale, q.shape[-2], cols)
    return q, scale


@torch.library.custom_op("primus_turbo::shuffle_mx_codes_impl", mutates_args=())
def _shuffle_codes_op(codes: torch.Tensor, inverse: bool) -> torch.Tensor:
    N.require_cuda(codes)
    _check(codes.dim() in (2, 3), "codes must be 2-D or 3-D")
    return _shuffle_codes_launch(codes.contiguous(), inverse)


@_shuffle_codes_op.register_fake
def _shuffle_codes_op_fake(codes, inverse):
    return torch.empty_like(codes)


def _mx_recipes(with_trans, scaling_recipe, scaling_recipe_for_trans, what):
    from primus_turbo.pytorch.core.low_precision import ScalingRecipe

    r = ScalingRecipe() if scaling_recipe is None else scaling_recipe
    rt = (ScalingRecipe() if scaling_recipe_for_trans is None else scaling_recipe_for_trans) if with_trans else r
    for rec in (r, rt):
        if (rec.use_rht or rec.use_sr) and what != "MXFP4":
            raise NotImplementedError(f"{what}: the Hadamard transform and stochastic rounding belong to the MXFP4 recipe")
        if rec.use_rht and rec.use_2d_block:
            raise NotImplementedError(f"{what}: the Hadamard transform is not combined with 2-D blocks")
    return r, rt


def _mx_flags(recipe) -> int:
    """Direction flags of the native quantizer: bit 0 = 2-D blocks, bit 1 = Hadamard transform,
    bit 2 = stochastic rounding."""
    if recipe is None:
        return 0
    return (1 if recipe.use_2d_block else 0) | (2 if recipe.use_rht else 0) | (4 if recipe.use_sr else 0)


_sr_counter = [0]


def _next_sr_seed(*flags: int) -> int:
    """A fresh 32-bit seed per stochastic-rounding launch (a process-wide counter, as the
    reference's quantizers keep one: reproducible for a fixed order of calls); 0 otherwise."""
    if not any(f & 4 for f in flags):
        return 0
    # The seed is a launch argument: a captured graph would replay the same rounding noise on
    # every step, which correlates the gradients' rounding errors. Refuse rather than do that.
    if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
        raise RuntimeError(
            "stochastic rounding (use_sr) cannot be captured into a HIP graph: its seed is a host-side launch "
            "argument and every replay would reuse it; quantize with use_sr outside the captured region"
        )
    _sr_counter[0] = (_sr_counter[0] + 1) & 0xFFFFFFFF
    return (_sr_counter[0] * 0x9E3779B1) & 0xFFFFFFFF


def _mx_check_axis(x, axis, with_trans):
    if not with_trans:
        if x.ndim == 2:
            assert axis in (0, 1), "The axis must be 0 or 1 when with_trans is False and x is 2D."
        elif x.ndim == 3:
            assert axis in (1, 2), "The axis must be 1 or 2 when with_trans is False and x is 3D."
        else:
            raise ValueError(f"The input tensor must be 2D or 3D but got {x.ndim}D.")
    else:
        assert axis is None, "The axis must be None when with_trans is True."
        assert x.ndim in (2, 3), f"The input tensor must be 2D or 3D but got {x.ndim}D."


def _mx_shapes(x, out_dtype, want_row, want_col):
    fp4 = _FP4X2 is not None and out_dtype == _FP4X2
    lead = tuple(x.shape[:-2])
    M, Nn = x.shape[-2], x.shape[-1]
    Mp, Np = -(-M // _MX_PAD) * _MX_PAD, -(-Nn // _MX_PAD) * _MX_PAD
    pack = 2 if fp4 else 1
    none = (0,)
    return (lead + (M, Np // pack) if want_row else none, lead + (M, Np // 32) if want_row else none,
            lead + (Nn, Mp // pack) if want_col else none, lead + (Nn, Mp // 32) if want_col else none)


def _mx_quantize(x: torch.Tensor, out_dtype: torch.dtype, want_row: bool, want_col: bool, row_flags: int, col_flags: int):
    """-> (row_q, row_scale, col_q, col_scale); the pair of an unwanted direction is None.
    ``row_flags`` / ``col_flags``: see ``_mx_flags``."""
    rq, rs, cq, cs = _quantize_mx_op(x, out_dtype, want_row, want_col, int(row_flags), int(col_flags))
    if not want_row:
        rq = rs = None
    if not want_col:
        cq = cs = None
    return rq, rs, cq, cs


@torch.library.custom_op("primus_turbo::quantize_mx", mutates_args=())
def _quantize_mx_op(x: torch.Tensor, out_dtype: torch.dtype, want_row: bool, want_col: bool, row_flags: int,
                    col_flags: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """The four outputs of ``_mx_quantize`` with an empty tensor for an unwanted direction (an
    operator returns tensors, not ``None``)."""
    N.require_cuda(x)
    if x.dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError("Input must be BFloat16 or Half")
    if not x.is_contiguous():
        raise RuntimeError("Input must be contiguous")
    fp4 = _FP4X2 is not None and out_dtype == _FP4X2
    if not fp4 and out_dtype not in (torch.float8_e4m3fn, torch.float8_e5m2):
        raise RuntimeError("Output must be Float8_e4m3fn, Float8_e5m2 or Float4_e2m1fn_x2")
    batched = x.dim() == 3
    B = x.shape[0] if batched else 1
    M, Nn = x.shape[-2], x.shape[-1]
    if Nn % 32 != 0:
        raise RuntimeError(f"N must be divisible by 32, got N={Nn}")
    Mp, Np = -(-M // _MX_PAD) * _MX_PAD, -(-Nn // _MX_PAD) * _MX_PAD
    pack = 2 if fp4 else 1
    lead = (B,) if batched else ()
    dev = x.device
    row_q = row_s = col_q = col_s = None
    if want_row:
        row_q = torch.empty(lead + (M, Np // pack), dtype=torch.uint8, device=dev)
        row_s = torch.empty(lead + (M, Np // 32), dtype=torch.uint8, device=dev)
    if want_col:
        col_q = torch.empty(lead + (Nn, Mp // pack), dtype=torch.uint8, device=dev)
        col_s = torch.empty(lead + (Nn, Mp // 32), dtype=torch.uint8, device=dev)
    N.check(
        N.lib().pt_quantize_mx(
            N.ptr(x), N.dtype_code(x.dtype), B, M, Nn, N.dtype_code(out_dtype),
            N.ptr(row_q), N.ptr(row_s), int(row_flags), N.ptr(col_q), N.ptr(col_s), int(col_flags),
            _next_sr_seed(row_flags if want_row else 0, col_flags if want_col else 0), N.stream_of(x),
        )
    )
    empty = lambda: torch.empty(0, dtype=torch.uint8, device=dev)  # noqa: E731
    view = lambda t, dt: (empty() if t is None else t).view(dt)  # noqa: E731
    return view(row_q, out_dtype), view(row_s, _E8M0), view(col_q, out_dtype), view(col_s, _E8M0)


@_quantize_mx_op.register_fake
def _quantize_mx_op_fake(x, out_dtype, want_row, want_col, row_flags, col_flags):
    shapes = _mx_shapes(x, out_dtype, want_row, want_col)
    mk = lambda shp, dt: torch.empty(shp, dtype=torch.uint8, device=x.device).view(dt)  # noqa: E731
    return mk(shapes[0], out_dtype), mk(shapes[1], _E8M0), mk(shapes[2], out_dtype), mk(shapes[3], _E8M0)


def _quantize_mx_impl(x, out_dtype, axis, block_size, with_trans, scaling_recipe, scaling_recipe_for_trans, what):
    assert block_size == 32, f"The block size must be 32 for {what} quantization"
    r, rt = _mx_recipes(with_trans, scaling_recipe, scaling_recipe_for_trans, what)
    _mx_check_axis(x, axis, with_trans)
    if with_trans:
        rq, rs, cq, cs = _mx_quantize(x, out_dtype, True, True, _mx_flags(r), _mx_flags(rt))
        return _apply_mx_shuffles(rq, rs, r, "rowwise") + _apply_mx_shuffles(cq, cs, rt, "colwise")
    rowwise = axis == x.ndim - 1
    rq, rs, cq, cs = _mx_quantize(x, out_dtype, rowwise, not rowwise, _mx_flags(r), _mx_flags(r))
    return _apply_mx_shuffles(rq, rs, r, "rowwise") if rowwise else _apply_mx_shuffles(cq, cs, r, "colwise")


def quantize_mxfp8_impl(x, out_dtype, axis, block_size, with_trans=False, scaling_recipe=None,
                        scaling_recipe_for_trans=None):
    """MXFP8 quantization. One direction (``axis``: last = along rows, else the transposed,
    column-direction output) -> ``(q, scale)``; ``with_trans`` -> ``(q_row, scale_row, q_col,
    scale_col)`` from a single read of ``x``. Shapes: row ``[.., M, N_pad]`` / ``[.., M, N_pad/32]``,
    col ``[.., N, M_pad]`` / ``[.., N, M_pad/32]`` with the pads rounding up to 128."""
    return _quantize_mx_impl(x, out_dtype, axis, block_size, with_trans, scaling_recipe, scaling_recipe_for_trans, "MXFP8")


def quantize_mxfp4_impl(x, out_dtype, axis, block_size, with_trans=False, scaling_recipe=None,
                        scaling_recipe_for_trans=None):
    """MXFP4 (E2M1, two codes per byte, even element in the low nibble); shapes as MXFP8 with
    the code tensors half as wide. ``use_rht`` in a recipe quantizes the values after the recipe's
    fixed 16-point Hadamard transform along that direction (1-D blocks only); ``use_sr`` rounds the
    codes stochastically (unbiased, a fresh seed per call; the scales stay deterministic)."""
    assert x.is_contiguous(), "The x tensor must be contiguous."
    return _quantize_mx_impl(x, out_dtype, axis, block_size, with_trans, scaling_recipe, scaling_recipe_for_trans, "MXFP4")


@torch.library.custom_op("primus_turbo::dequantize_mx", mutates_args=())
def _dequantize_mx_op(x: torch.Tensor, scale_inv: torch.Tensor, out_dtype: torch.dtype, rows: int, cols: int,
                      rowwise: bool) -> torch.Tensor:
    """``[rows, cols]`` codes with ``[rows, cols / 32]`` E8M0 scales -> ``[rows, cols]`` values, or
    their transpose ``[cols, rows]`` when not ``rowwise``."""
    out = torch.empty((rows, cols) if rowwise else (cols, rows), dtype=out_dtype, device=x.device)
    N.check(
        N.lib().pt_dequantize_mx(
            N.ptr(x), N.dtype_code(x.dtype), N.ptr(scale_inv), rows, cols, N.ptr(out), N.dtype_code(out_dtype),
            int(not rowwise), N.stream_of(x),
        )
    )
    return out


@_dequantize_mx_op.register_fake
def _dequantize_mx_op_fake(x, scale_inv, out_dtype, rows, cols, rowwise):
    return torch.empty((rows, cols) if rowwise else (cols, rows), dtype=out_dtype, device=x.device)


def _dequantize_mx(x, out_dtype, axis, block_size, scale_inv, fp4):
    assert x.is_contiguous(), "The x tensor must be contiguous."
    assert x.dim() in (2, 3), "The x must be a 2D or 3D tensor."
    assert scale_inv.dim() == x.dim(), "The scale_inv rank must match x."
    assert scale_inv.is_contiguous(), "The scale_inv tensor must be contiguous."
    if x.dim() == 2:
        assert axis in (0, 1), "The axis must be 0 or 1 for 2D input."
    else:
        assert axis in (1, 2), "The axis must be 1 or 2 for 3D input."
    assert out_dtype in (torch.float16, torch.bfloat16, torch.float32), f"unsupported out dtype {out_dtype}"
    assert block_size == 32
    N.require_cuda(x, scale_inv)
    rowwise = axis == x.dim() - 1
    rows = x.shape[0] if x.dim() == 2 else x.shape[0] * x.shape[1]
    cols = x.shape[-1] * (2 if fp4 else 1)
    assert cols % block_size == 0, "The last dimension of the x tensor must be divisible by the block size."
    assert scale_inv.numel() == rows * (cols // 32), "scale_inv does not match x"
    out = _dequantize_mx_op(x, scale_inv, out_dtype, rows, cols, rowwise)
    if x.dim() == 3:
        if rowwise:
            return out.reshape(x.shape[0], x.shape[1], cols)
        return out.reshape(cols, x.shape[0], x.shape[1]).permute(1, 2, 0)
    return out


def dequantize_mxfp8_impl(x, out_dtype, axis, block_size, scale_inv):
    """``y = float(q) * 2^(byte - 127)`` per 32-element block of the last axis; ``axis`` other
    than the last means ``x`` holds column-direction (transposed) data and the result is
    transposed back."""
    return _dequantize_mx(x, out_dtype, axis, block_size, scale_inv, fp4=False)


def dequantize_mxfp4_impl(x, out_dtype, axis, block_size, scale_inv):
    return _dequantize_mx(x, out_dtype, axis, block_size, scale_inv, fp4=True)


# ===========================================================================
# Grouped MXFP8 quantizers (MoE experts): per-group zero padding along M, 32 rows for the row
# direction and 128 for the transposed column direction
# ===========================================================================
MXFP8_GROUP_M_PADDING_ALIGN_SIZE = 32
MXFP8_K_DIM_PADDING_ALIGN_SIZE = 128


MXFP4_GROUP_K_DIM_PADDING_ALIGN_SIZE = 256


def _grouped_mx_quantize(x, out_dtype, group_lens, group_offs, want_row: bool, want_col: bool, row_flags: int = 0,
                         col_flags: int = 0):
    """MXFP8: rows of every group padded to 32, transposed columns to 128. MXFP4: rows stay
    where they are in ``x`` (their "padded" lens / offs are the originals), transposed columns
    padded to 256 per group.
    -> (row_q, row_scale, col_q, col_scale, lens_row, offs_row, lens_col, offs_col); the pair of an
    unwanted direction is None."""
    rq, rs, cq, cs, lr, orow, lc, ocol = _grouped_quantize_mx_op(x, out_dtype, group_lens, group_offs, want_row, want_col,
                                                                 int(row_flags), int(col_flags))
    if not want_row:
        rq = rs = None
    if not want_col:
        cq = cs = None
    if _FP4X2 is not None and out_dtype == _FP4X2:
        lr, orow = group_lens, group_offs
    return rq, rs, cq, cs, lr, orow, lc, ocol


def _grouped_mx_dims(M, Nn, G, fp4):
    ra = MXFP8_GROUP_M_PADDING_ALIGN_SIZE
    ca = MXFP4_GROUP_K_DIM_PADDING_ALIGN_SIZE if fp4 else MXFP8_K_DIM_PADDING_ALIGN_SIZE
    m_pad_row = M if fp4 else -(-(M + G * ra) // ra) * ra
    m_pad_col = -(-(M + G * ca) // ca) * ca
    n_pad = -(-Nn // _MX_PAD) * _MX_PAD
    return ra, ca, m_pad_row, m_pad_col, n_pad


@torch.library.custom_op("primus_turbo::grouped_quantize_mx", mutates_args=())
def _grouped_quantize_mx_op(
    x: torch.Tensor, out_dtype: torch.dtype, group_lens: torch.Tensor, group_offs: torch.Tensor, want_row: bool,
    want_col: bool, row_flags: int, col_flags: int,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """The outputs of ``_grouped_mx_quantize`` with an empty tensor where that returns None, and
    empty row lens / offs for MXFP4 (an operator may not hand its inputs back)."""
    N.require_cuda(x, group_lens, group_offs)
    if x.dtype not in (torch.bfloat16, torch.float16):
        raise RuntimeError("Input must be BFloat16 or Half")
    _check(x.dim() == 2 and x.is_contiguous(), "Input must be 2D and contiguous")
    _check(group_lens.dtype == torch.int64 and group_offs.dtype == torch.int64, "group_lens / group_offs must be int64")
    _check(group_lens.dim() == 1 and group_offs.dim() == 1 and group_offs.numel() == group_lens.numel() + 1,
           "group_offs.size(0) must equal group_lens.size(0) + 1")
    _check(group_lens.numel() >= 1, "must have at least one group")
    fp4 = _FP4X2 is not None and out_dtype == _FP4X2
    _check(fp4 or out_dtype in (torch.float8_e4m3fn, torch.float8_e5m2),
           "Output must be Float8_e4m3fn, Float8_e5m2 or Float4_e2m1fn_x2")
    M, Nn = x.shape
    _check(Nn % 32 == 0, f"N must be divisible by 32, got N={Nn}")
    G = group_lens.numel()
    pack = 2 if fp4 else 1
    ra, ca, m_pad_row, m_pad_col, n_pad = _grouped_mx_dims(M, Nn, G, fp4)
    dev = x.device
    group_offs = group_offs.contiguous()
    lens_row, offs_row = (group_lens, group_offs) if fp4 else _group_offs(group_lens, ra, True)
    lens_col, offs_col = _group_offs(group_lens, ca, True)
    row_q = row_s = col_q = col_s = None
    if want_row:
        row_q = torch.empty((m_pad_row, n_pad // pack), dtype=torch.uint8, device=dev)
        row_s = torch.empty((m_pad_row, n_pad // 32), dtype=torch.uint8, device=dev)
    if want_col:
        col_q = torch.empty((Nn, m_pad_col // pack), dtype=torch.uint8, device=dev)
        col_s = torch.empty((Nn, m_pad_col // 32), dtype=torch.uint8, device=dev)
    N.check(
        N.lib().pt_grouped_quantize_mx(
            N.ptr(x), N.dtype_code(x.dtype), M, Nn, N.dtype_code(out_dtype), N.ptr(group_offs),
            None if fp4 else N.ptr(offs_row), N.ptr(offs_col), G, N.ptr(row_q), N.ptr(row_s), int(row_flags), N.ptr(col_q),
            N.ptr(col_s), int(col_flags), m_pad_col,
            _next_sr_seed(row_flags if want_row else 0, col_flags if want_col else 0), N.stream_of(x),
        )
    )
    empty = lambda dt=torch.uint8: torch.empty(0, dtype=dt, device=dev)  # noqa: E731
    view = lambda t, dt: (empty() if t is None else t).view(dt)  # noqa: E731
    if fp4:
        lens_row, offs_row = empty(torch.int64), empty(torch.int64)
    return (view(row_q, out_dtype), view(row_s, _E8M0), view(col_q, out_dtype), view(col_s, _E8M0),
            lens_row, offs_row, lens_col, offs_col)


@_grouped_quantize_mx_op.register_fake
def _grouped_quantize_mx_op_fake(x, out_dtype, group_lens, group_offs, want_row, want_col, row_flags, col_flags):
    fp4 = _FP4X2 is not None and out_dtype == _FP4X2
    M, Nn = x.shape
    G = group_lens.numel()
    pack = 2 if fp4 else 1
    _, _, m_pad_row, m_pad_col, n_pad = _grouped_mx_dims(M, Nn, G, fp4)
    mk = lambda shp, dt: torch.empty(shp, dtype=torch.uint8, device=x.device).view(dt)  # noqa: E731
    i64 = lambda n: torch.empty(n, dtype=torch.int64, device=x.device)  # noqa: E731
    return (mk((m_pad_row, n_pad // pack) if want_row else (0,), out_dtype),
            mk((m_pad_row, n_pad // 32) if want_row else (0,), _E8M0),
            mk((Nn, m_pad_col // pack) if want_col else (0,), out_dtype),
            mk((Nn, m_pad_col // 32) if want_col else (0,), _E8M0),
            i64(0 if fp4 else G), i64(0 if fp4 else G + 1), i64(G), i64(G + 1))


@torch.library.custom_op("primus_turbo::glu_grouped_quantize_mx", mutates_args=())
def glu_grouped_quantize_mx_impl(
    x: torch.Tensor, probs: torch.Tensor, row_mask: Optional[torch.Tensor], act: str, out_dtype: torch.dtype,
    group_lens: torch.Tensor, group_offs: torch.Tensor, with_trans: bool, col_flags: int = 0,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Gated activation fused into the grouped MX quantizer: ``x [M, 2 N]`` is the fc1 output of an
    MoE expert MLP and the tensor quantized is ``y = T(act(x[:, :N]) * x[:, N:] * probs[:, None])``
    (zero rows where ``row_mask`` is 0), what ``swiglu_with_probs`` / ``geglu_with_probs`` would store,
    which never travels through HBM here. Outputs as ``primus_turbo::grouped_quantize_mx`` on the
    stored activation with round-to-nearest 1-D blocks, bit for bit: ``(row_q, row_scale, col_q,
    col_scale, lens_row, offs_row, lens_col, offs_col)``, the column pair empty unless ``with_trans``,
    row lens / offs empty for MXFP4 (its rows stay in place); ``col_flags=2`` transforms the MXFP4
    column direction (``use_rht``). (No counterpart in the reference.)"""
    N.require_cuda(x, probs, row_mask, group_lens, group_offs)
    _check(act in _GLU_ACT, "act must be 'silu' or 'gelu'")
    _check(x.dtype in (torch.bfloat16, torch.float16), "input must be bfloat16 or float16")
    _check(x.dim() == 2 and x.is_contiguous() and x.shape[1] % 2 == 0, "input must be a contiguous [M, 2 N] tensor")
    _check(group_lens.dtype == torch.int64 and group_offs.dtype == torch.int64, "group_lens / group_offs must be int64")
    _check(group_lens.dim() == 1 and group_offs.dim() == 1 and group_offs.numel() == group_lens.numel() + 1,
           "group_offs.size(0) must equal group_lens.size(0) + 1")
    _check(group_lens.numel() >= 1, "must have at least one group")
    fp4 = _FP4X2 is not None and out_dtype == _FP4X2
    _check(fp4 or out_dtype in (torch.float8_e4m3fn, torch.float8_e5m2),
           "Output must be Float8_e4m3fn, Float8_e5m2 or Float4_e2m1fn_x2")
    M, Nn = x.shape[0], x.shape[1] // 2
    _check(Nn % 32 == 0, f"N must be divisible by 32, got N={Nn}")
    _check(probs.numel() == M, "probs must hold one value per row")
    p32 = probs.reshape(-1).to(torch.float32).contiguous()
    mask = None
    if row_mask is not None:
        _check(row_mask.numel() == M, "row_mask must hold one value per row")
        mask = row_mask.reshape(-1).to(torch.int64).contiguous()
    G = group_lens.numel()
    pack = 2 if fp4 else 1
    ra, ca, m_pad_row, m_pad_col, n_pad = _grouped_mx_dims(M, Nn, G, fp4)
    dev = x.device
    group_offs = group_offs.contiguous()
    lens_row, offs_row = (group_lens, group_offs) if fp4 else _group_offs(group_lens, ra, True)
    lens_col, offs_col = _group_offs(group_lens, ca, True)
    row_q = torch.empty((m_pad_row, n_pad // pack), dtype=torch.uint8, device=dev)
    row_s = torch.empty((m_pad_row, n_pad // 32), dtype=torch.uint8, device=dev)
    col_q = col_s = None
    if with_trans:
        col_q = torch.empty((Nn, m_pad_col // pack), dtype=torch.uint8, device=dev)
        col_s = torch.empty((Nn, m_pad_col // 32), dtype=torch.uint8, device=dev)
    N.check(
        N.lib().pt_glu_grouped_quantize_mx(
            N.ptr(x), N.dtype_code(x.dtype), N.ptr(p32), N.ptr(mask), _GLU_ACT[act], M, Nn, N.dtype_code(out_dtype),
            N.ptr(group_offs), None if fp4 else N.ptr(offs_row), N.ptr(offs_col), G, N.ptr(row_q), N.ptr(row_s),
            N.ptr(col_q), N.ptr(col_s), int(col_flags) if with_trans else 0, m_pad_col, N.stream_of(x),
        )
    )
    empty = lambda dt=torch.uint8: torch.empty(0, dtype=dt, device=dev)  # noqa: E731
    view = lambda t, dt: (empty() if t is None else t).view(dt)  # noqa: E731
    if fp4:
        lens_row, offs_row = empty(torch.int64), empty(torch.int64)
    return (view(row_q, out_dtype), view(row_s, _E8M0), view(col_q, out_dtype), view(col_s, _E8M0),
            lens_row, offs_row, lens_col, offs_col)


@glu_grouped_quantize_mx_impl.register_fake
def _glu_grouped_quantize_mx_impl_fake(x, probs, row_mask, act, out_dtype, group_lens, group_offs, with_trans, col_flags=0):
    half = x.new_empty((x.shape[0], x.shape[1] // 2))
    return _grouped_quantize_mx_op_fake(half, out_dtype, group_lens, group_offs, True, with_trans, 0, 0)


def grouped_quantize_mxfp8_impl(x, out_dtype, axis, block_size, group_lens, group_offs, with_trans=False,
                                scaling_recipe=None, scaling_recipe_for_trans=None):
    """MXFP8 quantization of the packed rows of G groups, each virtually zero-padded along M.

    ``with_trans`` -> ``(row_q [M_pad_row, N_pad], row_scale [M_pad_row, N_pad/32], col_q [N, M_pad_col],
    col_scale [N, M_pad_col/32], lens_padded_row, offs_padded_row, lens_padded_col, offs_padded_col)``;
    otherwise ``(q, scale, group_lens_padded, group_offs_padded)`` of the direction ``axis`` asks
    for (1 = rows padded to 32 per group, 0 = transposed columns padded to 128 per group).
    ``M_pad_row`` / ``M_pad_col`` = ``total_M + G * align`` rounded up to ``align``; what lies
    beyond ``offs_padded[G]`` is unspecified."""
    assert block_size == 32, "The block size must be 32 for MXFP8 quantization"
    r, rt = _mx_recipes(with_trans, scaling_recipe, scaling_recipe_for_trans, "MXFP8")
    if with_trans:
        rq, rs, cq, cs, lr, orow, lc, ocol = _grouped_mx_quantize(x, out_dtype, group_lens, group_offs, True, True,
                                                                  _mx_flags(r), _mx_flags(rt))
        rq, rs = _apply_mx_shuffles(rq, rs, r, "rowwise")
        cq, cs = _apply_mx_shuffles(cq, cs, rt, "colwise")
        return rq, rs, cq, cs, lr, orow, lc, ocol
    assert axis in (0, 1), "The axis must be 0 or 1"
    rq, rs, cq, cs, lr, orow, lc, ocol = _grouped_mx_quantize(x, out_dtype, group_lens, group_offs, axis == 1, axis == 0,
                                                              _mx_flags(r), _mx_flags(r))
    if axis == 1:
        rq, rs = _apply_mx_shuffles(rq, rs, r, "rowwise")
        return rq, rs, lr, orow
    cq, cs = _apply_mx_shuffles(cq, cs, r, "colwise")
    return cq, cs, lc, ocol


def grouped_dequantize_mxfp8_impl(x, out_dtype, axis, block_size, scale_inv, group_offs, group_offs_padded,
                                  total_M=None):
    """Inverse of the grouped quantizer: the padded layout is de-quantized as a whole and the
    rows of every group are gathered back to their packed place (``[total_M, N]``). ``axis`` 1:
    ``x [M_pad_row, N_pad]``; 0: the transposed ``x [N, M_pad_col]``."""
    assert x.is_contiguous() and x.dim() == 2, "The x must be a contiguous 2D tensor."
    assert scale_inv.dim() == 2 and scale_inv.is_contiguous(), "The scale_inv must be a contiguous 2D tensor."
    assert axis in (0, 1), "The axis must be 0 or 1."
    full = _dequantize_mx(x, out_dtype, axis, block_size, scale_inv, fp4=False)  # [M_pad, N_pad]
    if total_M is None:
        total_M = int(group_offs[-1].item())
    # packed row i of group g sits at padded row i + (offs_padded[g] - offs[g])
    rows = torch.arange(total_M, device=x.device, dtype=torch.int64)
    g = torch.searchsorted(group_offs[1:].contiguous(), rows, right=True)
    src = rows + (group_offs_padded[:-1] - group_offs[:-1])[g]
    return full.index_select(0, src)


def grouped_quantize_mxfp4_impl(x, out_dtype, axis, block_size, group_lens, group_offs, with_trans=False,
                                scaling_recipe=None, scaling_recipe_for_trans=None):
    """MXFP4 quantization of the packed rows of G groups (reference: quantization_impl.py:657-811,
    layout of its default dispatch flydsl/quantization/mxfp4_grouped_quant.py:320-349).

    ``with_trans`` -> ``(row_q [M, N_pad/2], row_scale [M, N_pad/32], col_q [N, M_pad_col/2], col_scale
    [N, M_pad_col/32], group_lens, group_offs, lens_padded_col, offs_padded_col)``: the row
    direction keeps the rows where they are (row i = input row i), the transposed column
    direction pads every group to a multiple of 256 rows of zero data; ``M_pad_col`` = ``total_M +
    256 G`` rounded up to 256. Otherwise ``(q, scale, lens_padded, offs_padded)`` of the direction
    ``axis`` asks for (1 = rows, 0 = transposed columns). ``use_rht`` in a recipe applies the fixed
    16-point Hadamard transform along that direction (within each group's padded rows for the
    column direction), ``use_sr`` rounds the codes stochastically, ``use_2d_block`` shares one
    exponent per 32 x 32 block counted from the group's first row, ``shuffle_out`` /
    ``shuffle_scale`` give the pre-shuffled forms of the outputs (a pass over the plain ones)."""
    assert block_size == 32, "The block size must be 32 for MXFP4 quantization"
    assert _FP4X2 is not None and out_dtype == _FP4X2, "The out_dtype must be float4_e2m1fn_x2 for MXFP4 quantization"
    r, rt = _mx_recipes(with_trans, scaling_recipe, scaling_recipe_for_trans, "MXFP4")
    if with_trans:
        rq, rs, cq, cs, lr, orow, lc, ocol = _grouped_mx_quantize(x, out_dtype, group_lens, group_offs, True, True,
                                                                  _mx_flags(r), _mx_flags(rt))
        rq, rs = _apply_mx_shuffles(rq, rs, r, "rowwise")
        cq, cs = _apply_mx_shuffles(cq, cs, rt, "colwise")
        return rq, rs, cq, cs, lr, orow, lc, ocol
    assert axis in (0, 1), "The axis must be 0 (colwise) or 1 (rowwise) when with_trans is False."
    rq, rs, cq, cs, lr, orow, lc, ocol = _grouped_mx_quantize(x, out_dtype, group_lens, group_offs, axis == 1, axis == 0,
                                                              _mx_flags(r), _mx_flags(r))
    if axis == 1:
        rq, rs = _apply_mx_shuffles(rq, rs, r, "rowwise")
        return rq, rs, lr, orow
    cq, cs = _apply_mx_shuffles(cq, cs, r, "colwise")
    return cq, cs, lc, ocol
