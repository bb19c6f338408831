"""``QuantizedTensor``: a low-precision payload, its inverse scales and the recipe that made them,
presented to PyTorch as a tensor of the original shape and dtype.

Mirror of the reference's wrapper subclass (primus_turbo/pytorch/core/quantized_tensor.py:148-956):
same constructor keywords, factory, properties and private field names, the same handful of
tensor operations that work without de-quantizing (``view`` / ``reshape`` of the outer dimensions,
``detach``, ``select``, transposition), flatten / unflatten for ``torch.compile`` and FSDP, the
grouped (MoE, packed rows) variant with its padded offsets, and ``create_quantized_weight`` for
weight caches. Every kernel behind it is one of this library's quantizers.
"""

from __future__ import annotations

from typing import Any, Callable, Dict, NamedTuple, Optional, Tuple, Union

import torch

from primus_turbo import _native as N
from primus_turbo.pytorch.core.low_precision import (
    MXFP4_BLOCK_SIZE,
    MXFP8_BLOCK_SIZE,
    Float4QuantConfig,
    Float8QuantConfig,
    ScalingGranularity,
    ScalingRecipe,
    check_mxfp4_support,
    check_mxfp8_support,
    float4_e2m1fn_x2,
    float8_e4m3,
    float8_e5m2,
)

_G = ScalingGranularity
_FP8 = (float8_e4m3, float8_e5m2)
_SUPPORTED = tuple(d for d in (*_FP8, float4_e2m1fn_x2) if d is not None)
_MX_INNER_PAD = 128  # MX quantizers round the inner dimension of the payload up to this

# fields that travel unchanged through views, detach and flatten / unflatten
_META_FIELDS = ("_orig_dtype", "_dest_dtype", "_granularity", "_block_size", "_scaling_recipe", "_is_grouped_tensor",
                "_quantized_axis")
_GROUP_FIELDS = ("_orig_group_lens", "_orig_group_offs", "_group_lens", "_group_offs")


def _norm_axis(axis: Optional[int], ndim: int) -> Optional[int]:
    if axis is None:
        return None
    return axis if axis >= 0 else axis + ndim


def _is_fp4(dtype) -> bool:
    return float4_e2m1fn_x2 is not None and dtype == float4_e2m1fn_x2


@torch.library.custom_op("primus_turbo::transpose_last_two", mutates_args=())
def transpose_last_two(t: torch.Tensor) -> torch.Tensor:
    """Physical transpose of the last two dimensions of a contiguous 1-byte tensor (fp8 codes)."""
    assert t.element_size() == 1 and t.is_contiguous() and t.dim() in (2, 3)
    R, C = t.shape[-2], t.shape[-1]
    batch = t.shape[0] if t.dim() == 3 else 1
    out = torch.empty(t.shape[:-2] + (C, R), dtype=t.dtype, device=t.device)
    N.check(N.lib().pt_transpose_u8(N.ptr(t), N.ptr(out), batch, R, C, N.stream_of(t)))
    return out


@transpose_last_two.register_fake
def _transpose_last_two_fake(t):
    return torch.empty(tuple(t.shape[:-2]) + (t.shape[-1], t.shape[-2]), dtype=t.dtype, device=t.device)


class QuantizedTensor(torch.Tensor):
    """``shape`` / ``dtype`` describe the logical high-precision tensor, ``qdata`` / ``scale_inv`` /
    ``real_dtype`` what is stored. MX payloads are padded along their inner dimension; the
    wrapper keeps the unpadded shape and ``dequantize`` cuts the padding off again."""

    @staticmethod
    def __new__(cls, data: torch.Tensor, scale_inv: Optional[torch.Tensor], *, shape, orig_dtype: torch.dtype,
                dest_dtype: torch.dtype, granularity: ScalingGranularity,
                orig_group_lens: Optional[torch.Tensor] = None, orig_group_offs: Optional[torch.Tensor] = None,
                group_lens: Optional[torch.Tensor] = None, group_offs: Optional[torch.Tensor] = None,
                is_grouped_tensor: bool = False, block_size: Optional[int] = None,
                scaling_recipe: Optional[ScalingRecipe] = None, quantized_axis: Optional[int] = None,
                requires_grad: bool = False):
        assert dest_dtype in _SUPPORTED, "Unsupported quantized dtype"
        assert data.is_contiguous(), "data must be contiguous"
        assert scale_inv is not None and scale_inv.is_contiguous(), "scale_inv must be contiguous"
        self = torch.Tensor._make_wrapper_subclass(cls, torch.Size(shape), dtype=orig_dtype, layout=data.layout,
                                                   device=data.device, requires_grad=requires_grad)
        self._data, self._scale_inv = data, scale_inv
        self._orig_dtype, self._dest_dtype = orig_dtype, dest_dtype
        self._granularity, self._block_size = granularity, block_size
        self._scaling_recipe = scaling_recipe
        self._quantized_axis = quantized_axis
        self._is_grouped_tensor = is_grouped_tensor
        self._orig_group_lens, self._orig_group_offs = orig_group_lens, orig_group_offs
        self._group_lens, self._group_offs = group_lens, group_offs
        return self

    # ---------------------------------------------------------------- construction
    @staticmethod
    def _check_request(hp, dest_dtype, granularity, axis, grouped, block_size, scaling_recipe):
        assert hp.ndim in (2, 3), f"data must be a 2D or 3D tensor, got {hp.ndim}D"
        assert dest_dtype in _SUPPORTED, "Unsupported quantized dtype"
        if grouped:
            assert granularity in (_G.TENSORWISE, _G.ROWWISE, _G.MX_BLOCKWISE), f"Unsupported grouped granularity {granularity}"
            assert hp.ndim == 2, f"Grouped quantized tensor expects a 2D packed-M tensor, got {hp.ndim}D"
        else:
            assert granularity in (_G.TENSORWISE, _G.ROWWISE, _G.BLOCKWISE, _G.MX_BLOCKWISE), f"Unsupported granularity {granularity}"
        if _is_fp4(dest_dtype):
            assert granularity == _G.MX_BLOCKWISE, "FP4 only supports MX_BLOCKWISE granularity"
        if granularity == _G.BLOCKWISE:
            assert dest_dtype in _FP8, "Unsupported quantized dtype for BLOCKWISE"
            assert block_size is not None, "block_size must be provided for BLOCKWISE"
        if granularity == _G.MX_BLOCKWISE:
            ok, why = check_mxfp4_support() if _is_fp4(dest_dtype) else check_mxfp8_support()
            assert ok, why
            want = MXFP4_BLOCK_SIZE if _is_fp4(dest_dtype) else MXFP8_BLOCK_SIZE
            assert block_size == want, f"block_size must be {want} for MX_BLOCKWISE"
            assert scaling_recipe is not None, "scaling_recipe must be provided for MX_BLOCKWISE"
        if granularity != _G.TENSORWISE:
            assert axis is not None, "axis must be provided for non-TENSORWISE granularity"

    @classmethod
    def quantize(cls, hp_tensor: torch.Tensor, dest_dtype: torch.dtype, granularity: ScalingGranularity, *,
                 axis: Optional[int] = None, group_lens: Optional[torch.Tensor] = None,
                 block_size: Optional[int] = None, scaling_recipe: Optional[ScalingRecipe] = None) -> "QuantizedTensor":
        """Quantize ``hp_tensor`` (2-D, or 3-D stacked weights) along ``axis``. ``group_lens``
        marks the rows as the packed rows of MoE groups: MX_BLOCKWISE then uses the grouped
        quantizers (per-group padded layouts, ``group_lens`` / ``group_offs`` = the padded ones),
        TENSORWISE / ROWWISE quantize the packed rows as they are."""
        grouped = group_lens is not None
        cls._check_request(hp_tensor, dest_dtype, granularity, axis, grouped, block_size, scaling_recipe)
        x = hp_tensor.detach()
        if granularity in (_G.TENSORWISE, _G.ROWWISE):
            x = x.contiguous()
        kw: Dict[str, Any] = {}
        if grouped:
            from primus_turbo.pytorch.kernels.grouped_gemm.grouped_gemm_utils import group_offs_from_lens

            assert group_lens.is_cuda, "group_lens must be on CUDA"
            offs = group_offs_from_lens(group_lens)
            kw.update(orig_group_lens=group_lens, orig_group_offs=offs, is_grouped_tensor=True)
            if granularity == _G.MX_BLOCKWISE:
                data, scale, lens_p, offs_p = cls._grouped_quantize(x, dest_dtype, granularity, group_lens, offs, block_size,
                                                                    axis, scaling_recipe)
                kw.update(group_lens=lens_p, group_offs=offs_p)
            else:
                data, scale = cls._quantize(x, dest_dtype, granularity, block_size, axis, scaling_recipe)
                kw.update(group_lens=group_lens, group_offs=offs)
        else:
            data, scale = cls._quantize(x, dest_dtype, granularity, block_size, axis, scaling_recipe)
        return cls(data, scale, shape=hp_tensor.size(), orig_dtype=hp_tensor.dtype, dest_dtype=dest_dtype,
                   granularity=granularity, block_size=block_size, scaling_recipe=scaling_recipe, quantized_axis=axis,
                   requires_grad=hp_tensor.requires_grad, **kw)

    @classmethod
    @torch.no_grad()
    def _quantize(cls, x, dest_dtype, granularity, block_size=None, axis=None, scaling_recipe=None):
        from primus_turbo.pytorch.ops.quantization import quantize_fp4, quantize_fp8

        fn = quantize_fp4 if _is_fp4(dest_dtype) else quantize_fp8
        return fn(x, dest_dtype, granularity, block_size=block_size, axis=_norm_axis(axis, x.ndim),
                  scaling_recipe=scaling_recipe)

    @classmethod
    @torch.no_grad()
    def _grouped_quantize(cls, x, dest_dtype, granularity, group_lens, group_offs, block_size=None, axis=None,
                          scaling_recipe=None):
        from primus_turbo.pytorch.ops.quantization import grouped_quantize_fp4, grouped_quantize_fp8

        fn = grouped_quantize_fp4 if _is_fp4(dest_dtype) else grouped_quantize_fp8
        return fn(x, dest_dtype, granularity, group_lens, group_offs, block_size=block_size,
                  axis=_norm_axis(axis, x.ndim), scaling_recipe=scaling_recipe)

    # ---------------------------------------------------------------- accessors
    @property
    def qdata(self) -> torch.Tensor:
        return self._data

    @property
    def scale_inv(self) -> torch.Tensor:
        return self._scale_inv

    @property
    def group_lens(self) -> torch.Tensor:
        """Per-group row counts of the quantized layout (padded where the layout pads)."""
        assert self._is_grouped_tensor, "This is not a grouped tensor."
        return self._group_lens

    @property
    def group_offs(self) -> torch.Tensor:
        """Prefix sums of ``group_lens``: where each group starts in ``qdata``."""
        assert self._is_grouped_tensor, "This is not a grouped tensor."
        return self._group_offs

    @property
    def dtype(self) -> torch.dtype:  # type: ignore[override]
        return self._orig_dtype

    @property
    def real_dtype(self) -> torch.dtype:
        return self._dest_dtype

    @property
    def granularity(self) -> ScalingGranularity:
        return self._granularity

    @property
    def block_size(self) -> Optional[int]:
        return self._block_size

    @property
    def scaling_recipe(self) -> Optional[ScalingRecipe]:
        return self._scaling_recipe

    @property
    def quantized_axis(self) -> Optional[int]:
        return _norm_axis(self._quantized_axis, self._data.ndim)

    def __repr__(self, *, tensor_contents=None) -> str:
        gran = self._granularity.name if self._granularity is not None else None
        return (f"QuantizedTensor(shape={tuple(self.shape)}, dtype={self._orig_dtype}, real_dtype={self._dest_dtype}, "
                f"granularity={gran}, axis={self._quantized_axis}, block_size={self._block_size}, "
                f"grouped={self._is_grouped_tensor})")

    # ---------------------------------------------------------------- de-quantize
    @torch.no_grad()
    def dequantize(self) -> torch.Tensor:
        """Back to the original dtype and (unpadded) shape. Grouped MX layouts are gathered back
        to the packed rows."""
        from primus_turbo.pytorch.ops import quantization as Q

        axis = self.quantized_axis
        common = dict(block_size=self._block_size, axis=axis, scale_inv=self._scale_inv, scaling_recipe=self._scaling_recipe)
        fp4 = _is_fp4(self._dest_dtype)
        if self._is_grouped_tensor and self._granularity == _G.MX_BLOCKWISE:
            if fp4:
                out = Q.grouped_dequantize_fp4(self._data, self._orig_dtype, self._granularity, **common)
            else:
                assert self._group_offs is not None and self._orig_group_offs is not None, "group offsets are missing"
                out = Q.grouped_dequantize_fp8(self._data, self._orig_dtype, self._granularity, self._orig_group_offs,
                                               self._group_offs, total_M=self.shape[0], **common)
        else:
            fn = Q.dequantize_fp4 if fp4 else Q.dequantize_fp8
            out = fn(self._data, self._orig_dtype, self._granularity, **common)
        assert out.ndim in (2, 3), "Unsupported ndim"
        return out[..., : self.size(-1)].contiguous()

    # ---------------------------------------------------------------- flatten / unflatten
    def __tensor_flatten__(self):
        names = ["_data", "_scale_inv"] + [f for f in _GROUP_FIELDS if getattr(self, f) is not None]
        return names, {f: getattr(self, f) for f in _META_FIELDS}

    @staticmethod
    def __tensor_unflatten__(inner_tensors, metadata, outer_size, outer_stride):
        del outer_stride  # the wrapper is always contiguous
        return QuantizedTensor(
            inner_tensors["_data"], inner_tensors["_scale_inv"], shape=outer_size,
            orig_dtype=metadata["_orig_dtype"], dest_dtype=metadata["_dest_dtype"], granularity=metadata["_granularity"],
            block_size=metadata["_block_size"], scaling_recipe=metadata["_scaling_recipe"],
            is_grouped_tensor=metadata["_is_grouped_tensor"], quantized_axis=metadata.get("_quantized_axis"),
            orig_group_lens=inner_tensors.get("_orig_group_lens"), orig_group_offs=inner_tensors.get("_orig_group_offs"),
            group_lens=inner_tensors.get("_group_lens"), group_offs=inner_tensors.get("_group_offs"),
        )

    # ---------------------------------------------------------------- shape changes without de-quantizing
    @classmethod
    def _make_like(cls, tensor: "QuantizedTensor", *, data: torch.Tensor, scale_inv: torch.Tensor, shape) -> "QuantizedTensor":
        """A wrapper around other buffers with everything else (recipe, grouping) taken from ``tensor``."""
        return cls(data, scale_inv, shape=shape, orig_dtype=tensor._orig_dtype, dest_dtype=tensor._dest_dtype,
                   granularity=tensor._granularity, block_size=tensor._block_size, scaling_recipe=tensor._scaling_recipe,
                   orig_group_lens=tensor._orig_group_lens, orig_group_offs=tensor._orig_group_offs,
                   group_lens=tensor._group_lens, group_offs=tensor._group_offs,
                   is_grouped_tensor=tensor._is_grouped_tensor, quantized_axis=tensor._quantized_axis,
                   requires_grad=data.requires_grad)

    @staticmethod
    def _view_data_and_scale_inv(tensor: "QuantizedTensor", target_shape, op: Callable):
        """``op`` (``Tensor.view`` or ``Tensor.reshape``) applied to the payload and, for MX, to the
        scale bytes, for a logical target shape of the same rank. The payload's inner dimension
        is the logical one rounded up to the MX padding and divided by the codes per byte; other
        granularities keep their scale tensor as it is."""
        assert len(target_shape) == tensor._data.ndim, "views keep the rank of the quantized tensor"
        out_shape = torch.Size(target_shape)
        if out_shape == tensor.shape:
            return tensor._data, tensor._scale_inv, out_shape
        mx = tensor._granularity == _G.MX_BLOCKWISE
        pack = 2 if _is_fp4(tensor._dest_dtype) else 1
        inner = out_shape[-1]
        if mx:
            inner = -(-inner // _MX_INNER_PAD) * _MX_INNER_PAD
        assert inner % pack == 0, f"inner dimension {inner} must be divisible by {pack}"
        data = op(tensor._data, *out_shape[:-1], inner // pack)
        scale = tensor._scale_inv
        if mx and scale is not None:
            scale = op(scale, *out_shape[:-1], -(-inner // tensor._block_size))
        return data, scale, out_shape

    def view(self, *shape) -> "QuantizedTensor":
        return _ShapeFunc.apply(self, _flat_shape(shape), False)

    def reshape(self, *shape) -> "QuantizedTensor":
        return _ShapeFunc.apply(self, _flat_shape(shape), True)

    @classmethod
    def _transpose(cls, tensor: "QuantizedTensor", dim0: int, dim1: int) -> "QuantizedTensor":
        """TENSORWISE: the payload is transposed physically and shares the scalar scale. Other
        granularities cannot move their scales with the data: the tensor is de-quantized and
        quantized again along the other axis (the column-direction layout)."""
        nd = tensor.dim()
        d0, d1 = _norm_axis(dim0, nd), _norm_axis(dim1, nd)
        if d0 == d1:
            return cls._make_like(tensor, data=tensor._data, scale_inv=tensor._scale_inv, shape=tensor.shape)
        assert not tensor._is_grouped_tensor, "transpose is not supported for grouped QuantizedTensor"
        if tensor._granularity == _G.TENSORWISE:
            assert {d0, d1} == {nd - 2, nd - 1}, "only the last two dimensions can be exchanged"
            shape = list(tensor.shape)
            shape[d0], shape[d1] = shape[d1], shape[d0]
            return cls._make_like(tensor, data=transpose_last_two(tensor._data), scale_inv=tensor._scale_inv, shape=shape)
        return cls.quantize(tensor.dequantize(), tensor._dest_dtype, tensor._granularity, axis=-2,
                            block_size=tensor._block_size, scaling_recipe=tensor._scaling_recipe)

    # ---------------------------------------------------------------- dispatch
    @classmethod
    def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
        handler = _DISPATCH.get(func)
        if handler is not None and args and isinstance(args[0], QuantizedTensor):
            return handler(cls, func, args, kwargs or {})
        raise NotImplementedError(f"Unsupported dispatch: {func}")

    __torch_function__ = torch._C._disabled_torch_function_impl


def _flat_shape(shape) -> Tuple[int, ...]:
    if len(shape) == 1 and isinstance(shape[0], (tuple, list, torch.Size)):
        return tuple(shape[0])
    return tuple(shape)


def _d_view(cls, func, args, kwargs):
    d, s, shp = cls._view_data_and_scale_inv(args[0], args[1], torch.Tensor.view)
    return cls._make_like(args[0], data=d, scale_inv=s, shape=shp)


def _d_reshape(cls, func, args, kwargs):
    d, s, shp = cls._view_data_and_scale_inv(args[0], args[1], torch.Tensor.reshape)
    return cls._make_like(args[0], data=d, scale_inv=s, shape=shp)


def _d_select(cls, func, args, kwargs):
    return func(args[0]._data, *args[1:], **kwargs)  # a slice of the raw payload (e.g. one expert)


def _d_detach(cls, func, args, kwargs):
    t = args[0]
    return cls._make_like(t, data=t._data.detach(), scale_inv=t._scale_inv.detach(), shape=t.shape)


def _d_transpose(cls, func, args, kwargs):
    t = args[0]
    if func is torch.ops.aten.t.default:
        assert t.dim() == 2, "t() expects a 2D QuantizedTensor"
        return cls._transpose(t, 0, 1)
    return cls._transpose(t, args[1], args[2])


_DISPATCH = {
    torch.ops.aten.view.default: _d_view,
    torch.ops.aten._unsafe_view.default: _d_view,
    torch.ops.aten.reshape.default: _d_reshape,
    torch.ops.aten.select.int: _d_select,
    torch.ops.aten.detach.default: _d_detach,
    torch.ops.aten.alias.default: _d_detach,
    torch.ops.aten.t.default: _d_transpose,
    torch.ops.aten.transpose.int: _d_transpose,
}


class _ShapeFunc(torch.autograd.Function):
    """``view`` / ``reshape`` of a QuantizedTensor that autograd can see: the gradient (a plain
    tensor) takes the old shape back."""

    @staticmethod
    def forward(ctx, tensor: QuantizedTensor, shape: Tuple[int, ...], copy_ok: bool) -> QuantizedTensor:
        ctx.old_shape = tensor.shape
        op = torch.Tensor.reshape if copy_ok else torch.Tensor.view
        d, s, shp = QuantizedTensor._view_data_and_scale_inv(tensor, shape, op)
        return type(tensor)._make_like(tensor, data=d, scale_inv=s, shape=shp)

    @staticmethod
    def backward(ctx, grad):
        return grad.reshape(ctx.old_shape), None, None


class QuantizedTensorPair(NamedTuple):
    """A tensor quantized for the forward layout plus its counterpart for the backward layout."""

    data: QuantizedTensor
    data_t: Optional[QuantizedTensor] = None


def check_quantized_tensor(t: QuantizedTensor, config, axis: Optional[int] = None,
                           scaling_recipe: Optional[ScalingRecipe] = None) -> None:
    """Validate that a pre-quantized operand matches what the op would have produced. ``config``
    is anything with ``granularity`` and ``block_size``."""
    assert isinstance(t, QuantizedTensor)
    assert t.granularity == config.granularity, (
        f"QuantizedTensor granularity {t.granularity} does not match config granularity {config.granularity}"
    )
    if config.granularity in (_G.BLOCKWISE, _G.MX_BLOCKWISE):
        assert t.block_size == config.block_size, (
            f"QuantizedTensor block_size {t.block_size} does not match config block_size {config.block_size}"
        )
    if axis is not None and t.quantized_axis is not None:
        want = _norm_axis(axis, t.qdata.ndim)
        assert t.quantized_axis == want, f"QuantizedTensor quantized_axis {t.quantized_axis} does not match axis={want}"
    if scaling_recipe is not None:
        have = t.scaling_recipe if t.scaling_recipe is not None else ScalingRecipe()
        assert have == scaling_recipe, f"QuantizedTensor scaling_recipe {have} does not match {scaling_recipe}"


def _weight_recipe(cfg: Union[Float4QuantConfig, Float8QuantConfig]) -> ScalingRecipe:
    if isinstance(cfg, Float4QuantConfig):
        return ScalingRecipe(use_2d_block=True, shuffle_scale=cfg.use_preshuffle, shuffle_out=cfg.use_preshuffle)
    if cfg.granularity in (_G.BLOCKWISE, _G.MX_BLOCKWISE):
        return ScalingRecipe(use_2d_block=True)
    return ScalingRecipe()


def create_quantized_weight(weight, dest_dtype: torch.dtype, quant_config: Union[Float4QuantConfig, Float8QuantConfig],
                            need_weight_transpose_cache: bool = False
                            ) -> Tuple[QuantizedTensor, Optional[QuantizedTensor]]:
    """Quantize a weight once for reuse across micro-batches: the forward operand (along the last
    axis, square blocks where the granularity has blocks) and, on request, the operand that the
    backward product reads (reference: core/quantized_tensor.py:897-956). TENSORWISE transposes
    the payload; ROWWISE quantizes the transposed weight along its rows' other axis; block
    granularities quantize along axis -2, which stores the transposed layout."""
    recipe = _weight_recipe(quant_config)
    gran = quant_config.granularity
    kw = dict(dest_dtype=dest_dtype, granularity=gran, block_size=quant_config.block_size, scaling_recipe=recipe)
    qw = QuantizedTensor.quantize(weight, axis=-1, **kw)
    qw_t = None
    if need_weight_transpose_cache:
        if gran == _G.TENSORWISE:
            qw_t = qw.transpose(-2, -1)
        elif gran == _G.ROWWISE:
            qw_t = QuantizedTensor.quantize(weight.detach().transpose(-2, -1).contiguous(), axis=-2, **kw)
        elif gran in (_G.BLOCKWISE, _G.MX_BLOCKWISE):
            qw_t = QuantizedTensor.quantize(weight, axis=-2, **kw)
        else:
            raise ValueError(f"Unsupported granularity: {gran}")
    return qw, qw_t
