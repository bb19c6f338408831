"""The reference's MX dispatcher operators under their own names and schemas.

``torch.ops.primus_turbo_cpp_extension.quantize_mxfp8[_dual]``, ``quantize_mxfp4[_dual]``,
``dequantize_mxfp8`` / ``dequantize_mxfp4``, the grouped quantizers, ``grouped_dequantize_mxfp8`` and
``transpose_2d`` (csrc/pytorch/bindings_pytorch.cpp:44,52-93; argument checks and output shapes of
csrc/pytorch/quantization/quantization.cpp:285-359,436-969,971-1378 and
csrc/pytorch/transpose/transpose.cpp:17-49) as thin adapters over this library's MX entry points,
so that callers of the reference's extension module keep working. Each has a Meta implementation
for tracing.

Not offered (they raise ``NotImplementedError``): a ``padding_align_size`` other than 128, and the
Hadamard transform together with 2-D blocks.
"""

from __future__ import annotations

from typing import List, Optional

import torch

from primus_turbo import _native as N
from primus_turbo.pytorch.core.low_precision import ScalingRecipe
from primus_turbo.pytorch.kernels.quantization import quantization_impl as Q

_ext = Q._ext
_E8M0 = Q._E8M0
_FP4X2 = Q._FP4X2
_PAD = 128


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _pad_ok(padding_align_size: int) -> None:
    if padding_align_size != _PAD:
        raise NotImplementedError(f"MX quantization pads to {_PAD}; padding_align_size={padding_align_size} is not offered")


def _is_fp4(dtype) -> bool:
    return _FP4X2 is not None and dtype == _FP4X2


def _check_mx_in(x: torch.Tensor, dest_dtype, fp4: bool) -> None:
    N.require_cuda(x)
    _check(x.dim() in (2, 3), "Input must be 2D or 3D")
    _check(x.is_contiguous(), "Input must be contiguous")
    _check(x.dtype in (torch.bfloat16, torch.float16), "Input must be BFloat16 or Half")
    if fp4:
        _check(_is_fp4(dest_dtype), "Output must be Float4_e2m1fn_x2")
    else:
        _check(dest_dtype in (torch.float8_e4m3fn, torch.float8_e5m2), "Output must be Float8_e4m3fn or Float8_e5m2")


def _one_direction(x, dest_dtype, axis, recipe: ScalingRecipe, fp4: bool):
    _check_mx_in(x, dest_dtype, fp4)
    lo = x.dim() - 2
    _check(axis in (lo, lo + 1), f"Axis must be {lo} or {lo + 1} for {x.dim()}D input")
    fn = Q.quantize_mxfp4_impl if fp4 else Q.quantize_mxfp8_impl
    return list(fn(x, dest_dtype, axis, 32, False, recipe))


def _both_directions(x, dest_dtype, row: ScalingRecipe, col: ScalingRecipe, fp4: bool):
    _check_mx_in(x, dest_dtype, fp4)
    fn = Q.quantize_mxfp4_impl if fp4 else Q.quantize_mxfp8_impl
    return list(fn(x, dest_dtype, None, 32, True, row, col))


def _meta_pair(x, dest_dtype, rowwise: bool, fp4: bool, shuffle_scale: bool = False):
    shapes = Q._mx_shapes(x, dest_dtype, rowwise, not rowwise)
    q, s = (shapes[0], shapes[1]) if rowwise else (shapes[2], shapes[3])
    if shuffle_scale:  # the shuffled scale of every matrix is padded (shuffle_scale_batched)
        s = tuple(s[:-2]) + Q._scale_pad(s[-2], s[-1])
    mk = lambda shp, dt: torch.empty(shp, dtype=torch.uint8, device=x.device).view(dt)  # noqa: E731
    return [mk(q, dest_dtype), mk(s, _E8M0)]


# ---------------------------------------------------------------------------------------------
# dense quantizers
# ---------------------------------------------------------------------------------------------
_ext.define("quantize_mxfp8(Tensor input, ScalarType dest_dtype, int axis, int padding_align_size, "
            "bool use_2d_block, bool shuffle_scale=False, bool shuffle_out=False) -> Tensor[]")
_ext.define("quantize_mxfp8_dual(Tensor input, ScalarType dest_dtype, int padding_align_size, "
            "bool rowwise_use_2d_block, bool colwise_use_2d_block, "
            "bool shuffle_rowwise_scale=False, bool shuffle_rowwise=False, "
            "bool shuffle_colwise_scale=False, bool shuffle_colwise=False) -> Tensor[]")
_ext.define("quantize_mxfp4(Tensor input, ScalarType dest_dtype, int axis, int padding_align_size, "
            "bool use_2d_block, bool use_sr, bool use_rht, "
            "bool shuffle_scale=False, bool shuffle_out=False) -> Tensor[]")
_ext.define("quantize_mxfp4_dual(Tensor input, ScalarType dest_dtype, int padding_align_size, "
            "bool rowwise_use_2d_block, bool rowwise_use_sr, bool rowwise_use_rht, "
            "bool colwise_use_2d_block, bool colwise_use_sr, bool colwise_use_rht, "
            "bool shuffle_rowwise_scale=False, bool shuffle_rowwise=False, "
            "bool shuffle_colwise_scale=False, bool shuffle_colwise=False) -> Tensor[]")


def _quantize_mxfp8(input, dest_dtype, axis, padding_align_size, use_2d_block, shuffle_scale=False, shuffle_out=False):
    _pad_ok(padding_align_size)
    return _one_direction(input, dest_dtype, axis, ScalingRecipe(use_2d_block, False, False, shuffle_scale, shuffle_out), False)


def _quantize_mxfp8_meta(input, dest_dtype, axis, padding_align_size, use_2d_block, shuffle_scale=False, shuffle_out=False):
    return _meta_pair(input, dest_dtype, axis == input.dim() - 1, False, shuffle_scale)


def _quantize_mxfp8_dual(input, dest_dtype, padding_align_size, rowwise_use_2d_block, colwise_use_2d_block,
                         shuffle_rowwise_scale=False, shuffle_rowwise=False, shuffle_colwise_scale=False,
                         shuffle_colwise=False):
    _pad_ok(padding_align_size)
    return _both_directions(input, dest_dtype,
                            ScalingRecipe(rowwise_use_2d_block, False, False, shuffle_rowwise_scale, shuffle_rowwise),
                            ScalingRecipe(colwise_use_2d_block, False, False, shuffle_colwise_scale, shuffle_colwise), False)


def _quantize_mxfp8_dual_meta(input, dest_dtype, padding_align_size, rowwise_use_2d_block, colwise_use_2d_block,
                              shuffle_rowwise_scale=False, shuffle_rowwise=False, shuffle_colwise_scale=False,
                              shuffle_colwise=False):
    return (_meta_pair(input, dest_dtype, True, False, shuffle_rowwise_scale)
            + _meta_pair(input, dest_dtype, False, False, shuffle_colwise_scale))


def _quantize_mxfp4(input, dest_dtype, axis, padding_align_size, use_2d_block, use_sr, use_rht, shuffle_scale=False,
                    shuffle_out=False):
    _pad_ok(padding_align_size)
    return _one_direction(input, dest_dtype, axis, ScalingRecipe(use_2d_block, use_sr, use_rht, shuffle_scale, shuffle_out), True)


def _quantize_mxfp4_meta(input, dest_dtype, axis, padding_align_size, use_2d_block, use_sr, use_rht, shuffle_scale=False,
                         shuffle_out=False):
    return _meta_pair(input, dest_dtype, axis == input.dim() - 1, True, shuffle_scale)


def _quantize_mxfp4_dual(input, dest_dtype, padding_align_size, rowwise_use_2d_block, rowwise_use_sr, rowwise_use_rht,
                         colwise_use_2d_block, colwise_use_sr, colwise_use_rht, shuffle_rowwise_scale=False,
                         shuffle_rowwise=False, shuffle_colwise_scale=False, shuffle_colwise=False):
    _pad_ok(padding_align_size)
    return _both_directions(
        input, dest_dtype,
        ScalingRecipe(rowwise_use_2d_block, rowwise_use_sr, rowwise_use_rht, shuffle_rowwise_scale, shuffle_rowwise),
        ScalingRecipe(colwise_use_2d_block, colwise_use_sr, colwise_use_rht, shuffle_colwise_scale, shuffle_colwise), True)


def _quantize_mxfp4_dual_meta(input, dest_dtype, padding_align_size, rowwise_use_2d_block, rowwise_use_sr, rowwise_use_rht,
                              colwise_use_2d_block, colwise_use_sr, colwise_use_rht, shuffle_rowwise_scale=False,
                              shuffle_rowwise=False, shuffle_colwise_scale=False, shuffle_colwise=False):
    return (_meta_pair(input, dest_dtype, True, True, shuffle_rowwise_scale)
            + _meta_pair(input, dest_dtype, False, True, shuffle_colwise_scale))


# ---------------------------------------------------------------------------------------------
# dense de-quantizers
# ---------------------------------------------------------------------------------------------
_ext.define("dequantize_mxfp8(Tensor input, Tensor scale_inv, int axis, int block_size, ScalarType dest_dtype) -> Tensor")
_ext.define("dequantize_mxfp4(Tensor input, Tensor scale_inv, int axis, int block_size, ScalarType dest_dtype) -> Tensor")


def _check_dequant(input, scale_inv, axis, block_size, dest_dtype, fp4):
    N.require_cuda(input, scale_inv)
    _check(input.is_contiguous(), "Input must be contiguous")
    _check(input.dim() in (2, 3), "Input must be 2D or 3D")
    _check(_is_fp4(input.dtype) if fp4 else input.dtype in (torch.float8_e4m3fn, torch.float8_e5m2),
           "Input must be Float4_e2m1fn_x2" if fp4 else "Input must be FP8")
    _check(scale_inv.dim() == input.dim(), "scale_inv rank must match input")
    _check(scale_inv.is_contiguous(), "scale_inv must be contiguous")
    _check(scale_inv.dtype in (_E8M0, torch.uint8), "scale_inv must be Float8_e8m0fnu / uint8 tensor")
    _check(dest_dtype in (torch.bfloat16, torch.float16, torch.float32), "Output dtype must be bf16/fp16/fp32")
    _check(block_size == 32, "block_size must be 32")
    lo = input.dim() - 2
    _check(axis in (lo, lo + 1), f"Axis must be {lo} or {lo + 1} for {input.dim()}D input")


def _dequantize_mxfp8(input, scale_inv, axis, block_size, dest_dtype):
    _check_dequant(input, scale_inv, axis, block_size, dest_dtype, False)
    return Q.dequantize_mxfp8_impl(input, dest_dtype, axis, block_size, scale_inv.view(_E8M0))


def _dequantize_mxfp4(input, scale_inv, axis, block_size, dest_dtype):
    _check_dequant(input, scale_inv, axis, block_size, dest_dtype, True)
    return Q.dequantize_mxfp4_impl(input, dest_dtype, axis, block_size, scale_inv.view(_E8M0))


def _dequantize_mx_meta(fp4):
    def meta(input, scale_inv, axis, block_size, dest_dtype):
        pack = 2 if fp4 else 1
        rows, width = input.shape[-2], input.shape[-1] * pack
        lead = tuple(input.shape[:-2])
        rowwise = axis == input.dim() - 1
        return torch.empty(lead + ((rows, width) if rowwise else (width, rows)), dtype=dest_dtype, device=input.device)

    return meta


# ---------------------------------------------------------------------------------------------
# grouped quantizers
# ---------------------------------------------------------------------------------------------
_ext.define("grouped_quantize_mxfp8(Tensor input, Tensor group_lens, Tensor group_offs, ScalarType dest_dtype, int axis, "
            "int padding_align_size, bool use_2d_block, bool shuffle_scale=False, bool shuffle_out=False) -> Tensor[]")
_ext.define("grouped_quantize_mxfp8_dual(Tensor input, Tensor group_lens, Tensor group_offs, ScalarType dest_dtype, "
            "bool rowwise_use_2d_block, bool colwise_use_2d_block, "
            "bool shuffle_rowwise_scale=False, bool shuffle_rowwise=False, "
            "bool shuffle_colwise_scale=False, bool shuffle_colwise=False) -> Tensor[]")
_ext.define("grouped_quantize_mxfp4(Tensor input, Tensor group_lens, Tensor group_offs, ScalarType dest_dtype, int axis, "
            "bool use_2d_block, bool use_sr, bool use_rht) -> Tensor[]")
_ext.define("grouped_quantize_mxfp4_dual(Tensor input, Tensor group_lens, Tensor group_offs, ScalarType dest_dtype, "
            "bool rowwise_use_2d_block, bool rowwise_use_sr, bool rowwise_use_rht, "
            "bool colwise_use_2d_block, bool colwise_use_sr, bool colwise_use_rht) -> Tensor[]")
_ext.define("grouped_dequantize_mxfp8(Tensor input, Tensor scale_inv, Tensor group_offs, Tensor group_offs_padded, "
            "int axis, int block_size, ScalarType dest_dtype, int? total_M=None) -> Tensor")


def _check_grouped(input, group_lens, group_offs):
    N.require_cuda(input, group_lens, group_offs)
    _check(input.dim() == 2, "Input must be 2D")
    _check(input.is_contiguous(), "Input must be contiguous")
    _check(group_lens.dtype == torch.int64 and group_offs.dtype == torch.int64, "group tensors must be int64")
    _check(group_offs.numel() == group_lens.numel() + 1, "group_offs must have length G+1")


def _grouped_quantize_mxfp8(input, group_lens, group_offs, dest_dtype, axis, padding_align_size, use_2d_block,
                            shuffle_scale=False, shuffle_out=False):
    _pad_ok(padding_align_size)
    _check_grouped(input, group_lens, group_offs)
    _check(axis in (0, 1), "Axis must be 0 or 1")
    return list(Q.grouped_quantize_mxfp8_impl(input, dest_dtype, axis, 32, group_lens, group_offs, False,
                                              ScalingRecipe(use_2d_block, False, False, shuffle_scale, shuffle_out)))


def _grouped_quantize_mxfp8_dual(input, group_lens, group_offs, dest_dtype, rowwise_use_2d_block, colwise_use_2d_block,
                                 shuffle_rowwise_scale=False, shuffle_rowwise=False, shuffle_colwise_scale=False,
                                 shuffle_colwise=False):
    _check_grouped(input, group_lens, group_offs)
    return list(Q.grouped_quantize_mxfp8_impl(
        input, dest_dtype, None, 32, group_lens, group_offs, True,
        ScalingRecipe(rowwise_use_2d_block, False, False, shuffle_rowwise_scale, shuffle_rowwise),
        ScalingRecipe(colwise_use_2d_block, False, False, shuffle_colwise_scale, shuffle_colwise)))


def _grouped_quantize_mxfp4(input, group_lens, group_offs, dest_dtype, axis, use_2d_block, use_sr, use_rht):
    _check_grouped(input, group_lens, group_offs)
    _check(axis in (0, 1), "Axis must be 0 or 1")
    return list(Q.grouped_quantize_mxfp4_impl(input, dest_dtype, axis, 32, group_lens, group_offs, False,
                                              ScalingRecipe(use_2d_block, use_sr, use_rht)))


def _grouped_quantize_mxfp4_dual(input, group_lens, group_offs, dest_dtype, rowwise_use_2d_block, rowwise_use_sr,
                                 rowwise_use_rht, colwise_use_2d_block, colwise_use_sr, colwise_use_rht):
    _check_grouped(input, group_lens, group_offs)
    return list(Q.grouped_quantize_mxfp4_impl(input, dest_dtype, None, 32, group_lens, group_offs, True,
                                              ScalingRecipe(rowwise_use_2d_block, rowwise_use_sr, rowwise_use_rht),
                                              ScalingRecipe(colwise_use_2d_block, colwise_use_sr, colwise_use_rht)))


def _grouped_meta(fp4: bool, dual: bool):
    def meta(input, group_lens, group_offs, dest_dtype, *rest):
        M, Nn = input.shape
        G = group_lens.numel()
        _, _, m_pad_row, m_pad_col, n_pad = Q._grouped_mx_dims(M, Nn, G, fp4)
        pack = 2 if fp4 else 1
        dev = input.device
        mk = lambda shp, dt: torch.empty(shp, dtype=torch.uint8, device=dev).view(dt)  # noqa: E731
        lens = lambda: torch.empty(G, dtype=torch.int64, device=dev)  # noqa: E731
        offs = lambda: torch.empty(G + 1, dtype=torch.int64, device=dev)  # noqa: E731
        # the shuffle_scale arguments of the MXFP8 schemas (the MXFP4 ones have none)
        if fp4:
            shuf_row = shuf_col = False
        elif dual:
            shuf_row, shuf_col = (bool(rest[2]) if len(rest) > 2 else False), (bool(rest[4]) if len(rest) > 4 else False)
        else:
            shuf_row = shuf_col = bool(rest[3]) if len(rest) > 3 else False
        rs_shape = Q._scale_pad(m_pad_row, n_pad // 32) if shuf_row else (m_pad_row, n_pad // 32)
        cs_shape = Q._scale_pad(Nn, m_pad_col // 32) if shuf_col else (Nn, m_pad_col // 32)
        row = [mk((m_pad_row, n_pad // pack), dest_dtype), mk(rs_shape, _E8M0)]
        col = [mk((Nn, m_pad_col // pack), dest_dtype), mk(cs_shape, _E8M0)]
        if dual:
            return row + col + [lens(), offs(), lens(), offs()]
        axis = rest[0]
        return (row if axis == 1 else col) + [lens(), offs()]

    return meta


def _grouped_dequantize_mxfp8(input, scale_inv, group_offs, group_offs_padded, axis, block_size, dest_dtype,
                              total_M: Optional[int] = None):
    N.require_cuda(input, scale_inv, group_offs, group_offs_padded)
    _check(input.dim() == 2 and input.is_contiguous(), "Input must be a contiguous 2D tensor")
    _check(input.dtype in (torch.float8_e4m3fn, torch.float8_e5m2), "Input must be FP8")
    _check(scale_inv.dim() == 2 and scale_inv.is_contiguous(), "scale_inv must be a contiguous 2D tensor")
    _check(group_offs.dtype == torch.int64 and group_offs_padded.dtype == torch.int64, "group tensors must be int64")
    _check(group_offs.dim() == 1 and group_offs_padded.numel() == group_offs.numel() and group_offs.numel() >= 2,
           "group_offs / group_offs_padded must both have length G+1 (at least one group)")
    _check(axis in (0, 1), "Axis must be 0 or 1")
    _check(block_size == 32, "block_size must be 32")
    return Q.grouped_dequantize_mxfp8_impl(input, dest_dtype, axis, block_size, scale_inv.view(_E8M0), group_offs,
                                           group_offs_padded, total_M)


def _grouped_dequantize_mxfp8_meta(input, scale_inv, group_offs, group_offs_padded, axis, block_size, dest_dtype,
                                   total_M=None):
    if total_M is None:
        raise RuntimeError("grouped_dequantize_mxfp8 needs total_M to be traced (the row count is data otherwise)")
    n_cols = input.shape[1] if axis == 1 else input.shape[0]
    return torch.empty((total_M, n_cols), dtype=dest_dtype, device=input.device)


# ---------------------------------------------------------------------------------------------
# transpose_2d
# ---------------------------------------------------------------------------------------------
_ext.define("transpose_2d(Tensor input, int dim0, int dim1) -> Tensor")


def _transpose_dims(input, dim0, dim1):
    nd = input.dim()
    _check(nd in (2, 3), "transpose_2d only supports 2D or 3D input")
    d0, d1 = (dim0 if dim0 >= 0 else dim0 + nd), (dim1 if dim1 >= 0 else dim1 + nd)
    _check(0 <= d0 < nd and 0 <= d1 < nd, "transpose dim out of range")
    _check(min(d0, d1) == nd - 2 and max(d0, d1) == nd - 1,
           "transpose_2d only supports transposing the last two dims (-1, -2)")
    return tuple(input.shape[:-2]) + (input.shape[-1], input.shape[-2])


def _transpose_2d(input, dim0, dim1):
    N.require_cuda(input)
    _check(input.is_contiguous(), "input must be contiguous")
    shape = _transpose_dims(input, dim0, dim1)
    out = torch.empty(shape, dtype=input.dtype, device=input.device)
    if input.numel() == 0:
        return out
    batch = input.shape[0] if input.dim() == 3 else 1
    N.check(N.lib().pt_transpose_2d(N.ptr(input), N.ptr(out), batch, input.shape[-2], input.shape[-1],
                                    input.element_size(), N.stream_of(input)))
    return out


def _transpose_2d_meta(input, dim0, dim1):
    return torch.empty(_transpose_dims(input, dim0, dim1), dtype=input.dtype, device=input.device)


for _name, _fn, _meta in (
    ("quantize_mxfp8", _quantize_mxfp8, _quantize_mxfp8_meta),
    ("quantize_mxfp8_dual", _quantize_mxfp8_dual, _quantize_mxfp8_dual_meta),
    ("quantize_mxfp4", _quantize_mxfp4, _quantize_mxfp4_meta),
    ("quantize_mxfp4_dual", _quantize_mxfp4_dual, _quantize_mxfp4_dual_meta),
    ("dequantize_mxfp8", _dequantize_mxfp8, _dequantize_mx_meta(False)),
    ("dequantize_mxfp4", _dequantize_mxfp4, _dequantize_mx_meta(True)),
    ("grouped_quantize_mxfp8", _grouped_quantize_mxfp8, _grouped_meta(False, False)),
    ("grouped_quantize_mxfp8_dual", _grouped_quantize_mxfp8_dual, _grouped_meta(False, True)),
    ("grouped_quantize_mxfp4", _grouped_quantize_mxfp4, _grouped_meta(True, False)),
    ("grouped_quantize_mxfp4_dual", _grouped_quantize_mxfp4_dual, _grouped_meta(True, True)),
    ("grouped_dequantize_mxfp8", _grouped_dequantize_mxfp8, _grouped_dequantize_mxfp8_meta),
    ("transpose_2d", _transpose_2d, _transpose_2d_meta),
):
    _ext.impl(_name, _fn, "CUDA")
    _ext.impl(_name, _fn, "CPU")  # raises: there is no CPU path
    _ext.impl(_name, _meta, "Meta")
