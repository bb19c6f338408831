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


def _quantize_fp8_tensorwise(input: torch.Tensor, dest_dtype: torch.dtype, scale_opt: Optional[torch.Tensor] = None):
    N.require_cuda(input, scale_opt)
    _check(input.dtype in _HP_DTYPES, "input must be bfloat16, float16 or float32")
    _check_fp8_out(dest_dtype)
    _check(input.is_contiguous(), "input must be contiguous")
    lib = N.lib()
    out = torch.empty_like(input, dtype=dest_dtype)
    scale_inv = torch.empty((), dtype=torch.float32, device=input.device)
    ws = None
    scale_in = None
    if scale_opt is not None:
        _check(scale_opt.numel() == 1, "tensorwise scale must be scalar tensor")
        scale_in = scale_opt.to(torch.float32).contiguous()
    else:
        ws = N.zeroed_workspace(input.device, lib.pt_quantize_fp8_tensorwise_workspace_bytes(), "tw")
    N.check(
        lib.pt_quantize_fp8_tensorwise(
            N.ptr(input),
            N.dtype_code(input.dtype),
            input.numel(),
            N.ptr(out),
            N.dtype_code(dest_dtype),
            N.ptr(scale_in),
            N.ptr(scale_inv),
            N.ptr(ws),
            0 if ws is None else ws.numel(),
            N.stream_of(input),
        )
    )
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
