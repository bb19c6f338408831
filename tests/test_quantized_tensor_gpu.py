"""``QuantizedTensor`` as a tensor wrapper (cases of the reference's
tests/pytorch/core/test_quantized_tensor.py: construction and properties per granularity, the
constraints of ``quantize``, de-quantize round trips, flatten / unflatten, views of 2-D and 3-D
wrappers, grouped wrappers and their offsets), transposition, ``create_quantized_weight``, and
pre-quantized operands of the grouped MX GEMMs giving bit-identical results to quantizing inside
the op."""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, group_lens, to_f32_np
from oracle import gemm as OG

pytestmark = pytest.mark.gpu

M, N = 256, 512


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, QT, Pair, Recipe, F8, F4, E4M3, E5M2, FP4, create_quantized_weight, check_quantized_tensor, offs_from_lens
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig as F4
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig as F8
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.core.low_precision import ScalingRecipe as Recipe
    from primus_turbo.pytorch.core.low_precision import float4_e2m1fn_x2 as FP4
    from primus_turbo.pytorch.core.low_precision import float8_e4m3 as E4M3
    from primus_turbo.pytorch.core.low_precision import float8_e5m2 as E5M2
    from primus_turbo.pytorch.core.quantized_tensor import QuantizedTensor as QT
    from primus_turbo.pytorch.core.quantized_tensor import QuantizedTensorPair as Pair
    from primus_turbo.pytorch.core.quantized_tensor import check_quantized_tensor, create_quantized_weight
    from primus_turbo.pytorch.kernels.grouped_gemm.grouped_gemm_utils import group_offs_from_lens as offs_from_lens


CASES = ["tensorwise", "rowwise", "mxfp8", "mxfp4"]


def _spec(case):
    return {"tensorwise": (G.TENSORWISE, None, E4M3), "rowwise": (G.ROWWISE, None, E4M3),
            "mxfp8": (G.MX_BLOCKWISE, 32, E4M3), "mxfp4": (G.MX_BLOCKWISE, 32, FP4)}[case]


def _make(x, case, axis=-1, use_2d_block=False, lens=None):
    gran, bs, dt = _spec(case)
    kw = dict(axis=axis)
    if lens is not None:
        kw["group_lens"] = lens
    if gran == G.MX_BLOCKWISE:
        kw.update(block_size=bs, scaling_recipe=Recipe(use_2d_block=use_2d_block))
    return QT.quantize(x, dt, gran, **kw)


def _x(shape=(M, N), dtype=torch.bfloat16, seed=1):
    return bf16_randn(shape, seed=seed).to(dtype).cuda()


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_create_and_properties(case, dtype):
    gran, bs, dt = _spec(case)
    qt = _make(_x(dtype=dtype), case)
    assert isinstance(qt, torch.Tensor) and qt.dtype == dtype and qt.real_dtype == dt
    assert qt.shape == torch.Size([M, N]) and qt.device.type == "cuda" and qt.dim() == 2
    assert qt.granularity == gran and qt.block_size == bs and qt._is_grouped_tensor is False
    assert qt.quantized_axis == 1 and "QuantizedTensor" in repr(qt)
    want = {"tensorwise": (), "rowwise": (M, 1), "mxfp8": (M, N // 32), "mxfp4": (M, N // 32)}[case]
    assert tuple(qt.scale_inv.shape) == want
    assert tuple(qt.qdata.shape) == ((M, N // 2) if case == "mxfp4" else (M, N))
    with pytest.raises(AssertionError):
        qt.group_lens


def test_quantize_constraints():
    x = _x()
    with pytest.raises(AssertionError, match="scaling_recipe"):
        QT.quantize(x, E4M3, G.MX_BLOCKWISE, axis=-1, block_size=32)
    with pytest.raises(AssertionError, match="block_size"):
        QT.quantize(x, E4M3, G.MX_BLOCKWISE, axis=-1, block_size=128, scaling_recipe=Recipe())
    with pytest.raises(AssertionError, match="axis"):
        QT.quantize(x, E4M3, G.ROWWISE)
    with pytest.raises(AssertionError, match="2D or 3D"):
        QT.quantize(x.view(-1), E4M3, G.TENSORWISE)
    with pytest.raises(AssertionError, match="2D or 3D"):
        QT.quantize(x.view(2, 2, M // 4, N), E4M3, G.TENSORWISE)
    with pytest.raises(AssertionError, match="MX_BLOCKWISE"):
        QT.quantize(x, FP4, G.ROWWISE, axis=-1)
    with pytest.raises(AssertionError, match="2D packed-M"):
        QT.quantize(x.view(2, M // 2, N), E4M3, G.ROWWISE, axis=-1, group_lens=torch.tensor([M], device="cuda"))


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("shape", [(M, N), (200, 160), (3, 96, 224)])
def test_dequantize_round_trip(case, shape):
    x = _x(shape, seed=2)
    qt = _make(x, case)
    y = qt.dequantize()
    assert y.shape == x.shape and y.dtype == x.dtype
    assert OG.snr_db(to_f32_np(x), to_f32_np(y)) > (8 if case == "mxfp4" else 25)


@pytest.mark.parametrize("case", CASES)
def test_flatten_unflatten(case):
    qt = _make(_x(), case)
    names, meta = qt.__tensor_flatten__()
    assert names == ["_data", "_scale_inv"]
    rebuilt = QT.__tensor_unflatten__({n: getattr(qt, n) for n in names}, meta, qt.shape, qt.stride())
    assert rebuilt.shape == qt.shape and rebuilt.dtype == qt.dtype and rebuilt.real_dtype == qt.real_dtype
    assert rebuilt.granularity == qt.granularity and rebuilt.block_size == qt.block_size
    assert rebuilt.scaling_recipe == qt.scaling_recipe and rebuilt.quantized_axis == qt.quantized_axis
    assert rebuilt._data.data_ptr() == qt._data.data_ptr() and rebuilt._scale_inv.data_ptr() == qt._scale_inv.data_ptr()
    assert torch.equal(rebuilt.dequantize(), qt.dequantize())


@pytest.mark.parametrize("case", CASES)
def test_view_2d(case):
    qt = _make(_x(), case)
    for v in (qt.view(M, N), qt.reshape(M, N), qt.view((M, N))):
        assert v.shape == qt.shape and v._data.data_ptr() == qt._data.data_ptr()
        assert v._scale_inv.data_ptr() == qt._scale_inv.data_ptr()
        for f in ("_granularity", "_block_size", "_orig_dtype", "_dest_dtype", "_scaling_recipe", "_is_grouped_tensor"):
            assert getattr(v, f) == getattr(qt, f)
    with pytest.raises(AssertionError):
        qt.view(M * N)  # rank changes are not views of the payload
    d = qt.detach()
    assert isinstance(d, QT) and d._data.data_ptr() == qt._data.data_ptr() and not d.requires_grad


@pytest.mark.parametrize("case", ["tensorwise", "mxfp8", "mxfp4"])
def test_view_3d_regroups_rows(case):
    """[G, R, K] <-> [G * R / 2, 2, K]-style regrouping of the outer dimensions keeps the payload."""
    Gn, R, K = 4, 64, 256
    x = _x((Gn, R, K), seed=3)
    qt = _make(x, case)
    v = qt.view(Gn * 2, R // 2, K)
    assert v.shape == (Gn * 2, R // 2, K) and v._data.data_ptr() == qt._data.data_ptr()
    assert torch.equal(v.dequantize(), qt.dequantize().view(Gn * 2, R // 2, K))
    assert torch.equal(v.reshape(Gn, R, K).dequantize(), qt.dequantize())
    # select hands out the raw payload of one slice
    assert torch.equal(qt[1].view(torch.uint8), qt.qdata[1].view(torch.uint8))


def test_view_is_visible_to_autograd():
    w = torch.nn.Parameter(_x((4, 64, 256), seed=4))
    qt = _make(w, "tensorwise")
    assert qt.requires_grad
    v = qt.view(8, 32, 256)
    assert v.grad_fn is not None


def test_transpose():
    x = _x((200, 160), seed=5)
    qt = _make(x, "tensorwise")
    for t in (qt.t(), qt.transpose(0, 1), qt.transpose(-1, -2)):
        assert t.shape == (160, 200) and t.scale_inv.data_ptr() == qt.scale_inv.data_ptr()
        assert torch.equal(t.qdata.view(torch.uint8), qt.qdata.view(torch.uint8).t().contiguous())
        assert torch.equal(t.dequantize(), qt.dequantize().t())
    assert qt.transpose(1, 1)._data.data_ptr() == qt._data.data_ptr()
    x3 = _x((3, 64, 96), seed=6)
    q3 = _make(x3, "tensorwise")
    assert torch.equal(q3.transpose(-2, -1).dequantize(), q3.dequantize().transpose(-2, -1))
    # scaled rows cannot follow the data: the other axis is quantized afresh
    r = _make(x, "rowwise").transpose(0, 1)
    assert r.quantized_axis == 0 and tuple(r.scale_inv.shape) == (1, 160)
    m = _make(_x((256, 128), seed=7), "mxfp8").t()
    assert m.quantized_axis == 0 and tuple(m.qdata.shape) == (128, 256)


LENS = [64, 64, 64, 64]


@pytest.mark.parametrize("case", ["tensorwise", "rowwise"])
@pytest.mark.parametrize("lens", [LENS, [20, 80, 60, 96]])
def test_grouped_plain_granularities(case, lens):
    """TENSORWISE / ROWWISE treat the packed rows as one tensor and only carry the offsets."""
    gl = torch.tensor(lens, dtype=torch.int64, device="cuda")
    x = _x()
    qt = _make(x, case, lens=gl)
    plain = _make(x, case)
    assert qt._is_grouped_tensor is True and qt.shape == (M, N)
    assert torch.equal(qt._orig_group_lens, gl) and torch.equal(qt._orig_group_offs, offs_from_lens(gl))
    assert torch.equal(qt.group_lens, gl) and torch.equal(qt.group_offs, offs_from_lens(gl))
    assert torch.equal(qt.qdata.view(torch.uint8), plain.qdata.view(torch.uint8)) and torch.equal(qt.scale_inv, plain.scale_inv)
    assert torch.equal(qt.dequantize(), plain.dequantize())
    names, meta = qt.__tensor_flatten__()
    assert set(names) == {"_data", "_scale_inv", "_orig_group_lens", "_orig_group_offs", "_group_lens", "_group_offs"}
    rebuilt = QT.__tensor_unflatten__({n: getattr(qt, n) for n in names}, meta, qt.shape, qt.stride())
    assert rebuilt._is_grouped_tensor and torch.equal(rebuilt.group_offs, qt.group_offs)
    v = qt.view(M, N)
    assert v._is_grouped_tensor and v.group_offs is qt.group_offs
    with pytest.raises(AssertionError, match="grouped"):
        qt.t()


@pytest.mark.parametrize("case", ["mxfp8", "mxfp4"])
@pytest.mark.parametrize("axis", [-1, -2])
def test_grouped_mx(case, axis):
    lens = group_lens("ragged", 4, 500, 8)
    gl = torch.from_numpy(lens).cuda()
    x = _x((500, 160), seed=9)
    qt = _make(x, case, axis=axis, lens=gl)
    assert qt._is_grouped_tensor and qt.shape == (500, 160) and qt.quantized_axis == (1 if axis == -1 else 0)
    align = {("mxfp8", -1): 32, ("mxfp8", -2): 128, ("mxfp4", -1): 1, ("mxfp4", -2): 256}[(case, axis)]
    want = (lens + align - 1) // align * align
    assert np.array_equal(qt.group_lens.cpu().numpy(), want)
    assert np.array_equal(qt.group_offs.cpu().numpy(), np.concatenate([[0], np.cumsum(want)]))
    if not (case == "mxfp4" and axis == -2):  # the FP4 column direction has no gathering de-quantizer
        y = qt.dequantize()
        assert y.shape == x.shape and OG.snr_db(to_f32_np(x), to_f32_np(y)) > (8 if case == "mxfp4" else 25)


@pytest.mark.parametrize("gran,cfg", [("tensorwise", None), ("rowwise", None), ("blockwise", None), ("mxfp8", None), ("mxfp4", None)])
def test_create_quantized_weight(gran, cfg):
    w = _x((384, 256), seed=10)
    if gran == "mxfp4":
        cfg, dt = F4(), FP4
    else:
        from primus_turbo.pytorch.core.low_precision import ScaleDtype
        g = {"tensorwise": G.TENSORWISE, "rowwise": G.ROWWISE, "blockwise": G.BLOCKWISE, "mxfp8": G.MX_BLOCKWISE}[gran]
        cfg = F8(granularity=g, block_size={"blockwise": 128, "mxfp8": 32}.get(gran),
                 **({"scale_dtype": ScaleDtype.E8M0} if gran == "mxfp8" else {}))
        dt = E4M3
    qw, none = create_quantized_weight(w, dt, cfg)
    assert none is None and qw.shape == w.shape and qw.quantized_axis == 1
    check_quantized_tensor(qw, cfg, axis=-1)
    qw2, qw_t = create_quantized_weight(w, dt, cfg, need_weight_transpose_cache=True)
    assert torch.equal(qw2.qdata.view(torch.uint8), qw.qdata.view(torch.uint8))
    assert isinstance(qw_t, QT)
    gate = 8 if gran == "mxfp4" else 25
    assert OG.snr_db(to_f32_np(w), to_f32_np(qw.dequantize())) > gate
    back = qw_t.dequantize()
    back = back.t() if back.shape != w.shape else back
    assert OG.snr_db(to_f32_np(w), to_f32_np(back)) > gate
    # the cached pair drives the dense op to the same result as quantizing inside it
    a = _x((128, 256), seed=11).requires_grad_(True)
    op = turbo.ops.gemm_fp4 if gran == "mxfp4" else turbo.ops.gemm_fp8
    y_ref = op(a, w, trans_b=True, config=cfg)
    # (ROWWISE caches the transposed weight, which the dense op does not read: it wants the weight
    # in place, quantized along its other axis)
    y = op(a, Pair(qw2, None if gran == "rowwise" else qw_t), trans_b=True, config=cfg)
    assert torch.equal(y, y_ref)


@pytest.mark.parametrize("case", ["mxfp8", "mxfp4"])
def test_grouped_gemm_prequantized_operands(case):
    """Grouped MX GEMMs with a grouped QuantizedTensor activation and a cached weight pair: forward
    and both gradients are bit-identical to the op quantizing its own operands."""
    from primus_turbo.pytorch.core.low_precision import Format, ScaleDtype

    lens = group_lens("ragged", 4, 1000, 12)
    gl = torch.from_numpy(lens).cuda()
    K, Nn = 1024, 512
    a = _x((1000, K), seed=13)
    w = _x((4, Nn, K), seed=14)
    dy = _x((1000, Nn), seed=15)
    if case == "mxfp4":
        cfg, dt, op = F4(), FP4, turbo.ops.grouped_gemm_fp4
    else:
        cfg = F8(format=Format.E4M3, granularity=G.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0)
        dt, op = E4M3, turbo.ops.grouped_gemm_fp8
    a1, w1 = a.clone().requires_grad_(True), w.clone().requires_grad_(True)
    y_ref = op(a1, w1, gl, trans_b=True, config=cfg)
    y_ref.backward(dy)
    qa = QT.quantize(a, dt, G.MX_BLOCKWISE, axis=-1, group_lens=gl, block_size=32, scaling_recipe=Recipe())
    # (the MXFP4 recipe puts the Hadamard transform on the wgrad operands)
    qa_t = QT.quantize(a, dt, G.MX_BLOCKWISE, axis=-2, group_lens=gl, block_size=32,
                       scaling_recipe=Recipe(use_rht=(case == "mxfp4")))
    qw, qw_t = create_quantized_weight(w, dt, cfg, need_weight_transpose_cache=True)
    with torch.no_grad():
        assert torch.equal(op(qa, qw, gl, trans_b=True, config=cfg), y_ref)
        assert torch.equal(op(Pair(qa, qa_t), Pair(qw, qw_t), gl, trans_b=True, config=cfg), y_ref)
    # gradients through the cached pair (the weight wrapper is the leaf here)
    w2 = torch.nn.Parameter(w.clone())
    qw2, qw2_t = create_quantized_weight(w2, dt, cfg, need_weight_transpose_cache=True)
    a2 = a.clone().requires_grad_(True)
    y = op(a2, Pair(qw2, qw2_t), gl, trans_b=True, config=cfg)
    assert torch.equal(y, y_ref)
    y.backward(dy)
    assert torch.equal(a2.grad, a1.grad)
    assert qw2.grad is not None and torch.equal(qw2.grad, w1.grad)
