"""Host-side behaviour of the ``QuantizedTensor`` wrapper on hand-made CPU buffers (no kernel is
called): what it reports to PyTorch, views of the outer dimensions with MX padding and FP4 packing,
flatten / unflatten, grouped bookkeeping, and the checks of ``check_quantized_tensor``."""

import pytest
import torch

from primus_turbo.pytorch.core.low_precision import (
    Float8QuantConfig,
    ScalingGranularity as G,
    ScalingRecipe,
    float4_e2m1fn_x2,
    float8_e4m3,
)
from primus_turbo.pytorch.core.quantized_tensor import QuantizedTensor as QT
from primus_turbo.pytorch.core.quantized_tensor import check_quantized_tensor


def _wrap(shape, gran, dest=float8_e4m3, block=None, recipe=None, axis=-1, **kw):
    inner = shape[-1]
    pack = 2 if dest == float4_e2m1fn_x2 else 1
    if gran == G.MX_BLOCKWISE:
        inner = -(-inner // 128) * 128
    data = torch.arange(int(torch.tensor(shape[:-1]).prod()) * (inner // pack), dtype=torch.int64).to(torch.uint8)
    data = data.view(*shape[:-1], inner // pack).view(dest)
    if gran == G.TENSORWISE:
        scale = torch.ones(())
    elif gran == G.ROWWISE:
        scale = torch.ones(*shape[:-1], 1)
    else:
        scale = torch.arange(int(torch.tensor(shape[:-1]).prod()) * (inner // 32)).to(torch.uint8).view(*shape[:-1], inner // 32)
    return QT(data, scale, shape=shape, orig_dtype=torch.bfloat16, dest_dtype=dest, granularity=gran, block_size=block,
              scaling_recipe=recipe, quantized_axis=axis, **kw)


def test_reports_the_logical_tensor():
    q = _wrap((4, 160), G.MX_BLOCKWISE, block=32, recipe=ScalingRecipe())
    assert isinstance(q, torch.Tensor) and q.shape == (4, 160) and q.dtype == torch.bfloat16
    assert q.real_dtype == float8_e4m3 and tuple(q.qdata.shape) == (4, 256) and tuple(q.scale_inv.shape) == (4, 8)
    assert q.quantized_axis == 1 and q.is_contiguous() and q.dim() == 2 and not q.requires_grad
    assert "MX_BLOCKWISE" in repr(q)
    with pytest.raises(NotImplementedError):
        q + 1  # arithmetic needs an explicit dequantize()
    with pytest.raises(AssertionError):
        QT(q.qdata.t(), q.scale_inv, shape=(256, 4), orig_dtype=torch.bfloat16, dest_dtype=float8_e4m3,
           granularity=G.TENSORWISE)  # non-contiguous payload


@pytest.mark.parametrize("dest", [float8_e4m3, float4_e2m1fn_x2])
def test_views_regroup_outer_dims_of_mx_payloads(dest):
    q = _wrap((4, 6, 160), G.MX_BLOCKWISE, dest=dest, block=32, recipe=ScalingRecipe())
    pack = 2 if dest == float4_e2m1fn_x2 else 1
    v = q.view(8, 3, 160)
    assert v.shape == (8, 3, 160) and tuple(v.qdata.shape) == (8, 3, 256 // pack) and tuple(v.scale_inv.shape) == (8, 3, 8)
    assert v.qdata.data_ptr() == q.qdata.data_ptr() and v.scale_inv.data_ptr() == q.scale_inv.data_ptr()
    assert torch.equal(v.qdata.view(torch.uint8).reshape(-1), q.qdata.view(torch.uint8).reshape(-1))
    r = q.reshape(2, 12, 160)
    assert tuple(r.qdata.shape) == (2, 12, 256 // pack) and r.block_size == 32 and r.scaling_recipe == ScalingRecipe()
    assert q.view(4, 6, 160).qdata.data_ptr() == q.qdata.data_ptr()
    with pytest.raises(AssertionError):
        q.view(24, 160)
    assert torch.equal(q[2].view(torch.uint8), q.qdata[2].view(torch.uint8))


def test_rowwise_view_keeps_scale_tensor():
    q = _wrap((4, 6, 64), G.ROWWISE)
    v = q.view(2, 12, 64)
    assert v.scale_inv is q.scale_inv and tuple(v.qdata.shape) == (2, 12, 64)


def test_flatten_round_trip_with_groups():
    lens = torch.tensor([3, 0, 5]); offs = torch.tensor([0, 3, 3, 8])
    q = _wrap((8, 64), G.ROWWISE, orig_group_lens=lens, orig_group_offs=offs, group_lens=lens, group_offs=offs,
              is_grouped_tensor=True)
    names, meta = q.__tensor_flatten__()
    assert names == ["_data", "_scale_inv", "_orig_group_lens", "_orig_group_offs", "_group_lens", "_group_offs"]
    back = QT.__tensor_unflatten__({n: getattr(q, n) for n in names}, meta, q.shape, q.stride())
    assert back._is_grouped_tensor and back.group_offs is offs and back.granularity == G.ROWWISE and back.shape == q.shape
    d = q.detach()
    assert d._is_grouped_tensor and d.group_lens is lens
    with pytest.raises(AssertionError, match="grouped"):
        q.t()
    plain = _wrap((8, 64), G.ROWWISE)
    with pytest.raises(AssertionError, match="not a grouped"):
        plain.group_offs


def test_check_quantized_tensor():
    cfg = Float8QuantConfig(granularity=G.BLOCKWISE, block_size=128)
    q = _wrap((4, 256), G.BLOCKWISE, block=128, recipe=ScalingRecipe(use_2d_block=True))
    check_quantized_tensor(q, cfg, axis=-1, scaling_recipe=ScalingRecipe(use_2d_block=True))
    with pytest.raises(AssertionError, match="granularity"):
        check_quantized_tensor(q, Float8QuantConfig(granularity=G.ROWWISE))
    with pytest.raises(AssertionError, match="axis"):
        check_quantized_tensor(q, cfg, axis=-2)
    with pytest.raises(AssertionError, match="scaling_recipe"):
        check_quantized_tensor(q, cfg, scaling_recipe=ScalingRecipe())
    with pytest.raises(AssertionError, match="block_size"):
        check_quantized_tensor(_wrap((4, 256), G.BLOCKWISE, block=64), cfg)
