"""Every op family traces into ONE graph under ``torch.compile(fullgraph=True)``: each native
launch sits behind a registered operator with a shape function, so Dynamo never meets a raw
pointer or a stream handle. Traced on ``meta`` tensors with the ``aot_eager`` backend, which runs
the shape functions only: no GPU is needed, and what is checked is the shapes and dtypes of
outputs and gradients. (The reference compiles its FP8 linear layer with ``fullgraph=False``,
tests/pytorch/modules/test_linear_fp8.py:33-70, and switches Dynamo off around gemm_fp8 / gemm_fp4 /
grouped_gemm_fp4, ops/gemm_fp8.py:720; results under compilation are compared on the GPU in
test_torch_compile_gpu.py.)"""

import pytest
import torch


@pytest.fixture(scope="module")
def turbo(native_lib):
    import primus_turbo.pytorch as turbo
    import primus_turbo.pytorch.core.low_precision as LP

    saved = LP._needs
    LP._needs = lambda *a: (True, "")  # the hardware check looks for a gfx950 device; tracing needs none
    yield turbo
    LP._needs = saved


def _cfg(name):
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, ScaleDtype, ScalingGranularity as G

    return {
        "tensorwise": lambda: Float8QuantConfig(granularity=G.TENSORWISE),
        "rowwise": lambda: Float8QuantConfig(granularity=G.ROWWISE),
        "blockwise": lambda: Float8QuantConfig(granularity=G.BLOCKWISE, block_size=128),
        "mx": lambda: Float8QuantConfig(granularity=G.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0),
    }[name]()


def _meta(*shape, dtype=torch.bfloat16, grad=True):
    return torch.empty(*shape, device="meta", dtype=dtype, requires_grad=grad)


def _trace(fn, *args):
    torch._dynamo.reset()
    out = torch.compile(fn, fullgraph=True, backend="aot_eager")(*args)
    out.sum().backward()
    return out


GRANS = ["tensorwise", "rowwise", "blockwise", "mx"]


@pytest.mark.parametrize("gran", GRANS)
def test_gemm_fp8_traces_fullgraph(turbo, gran):
    cfg = _cfg(gran)
    a, b = _meta(256, 512), _meta(384, 512)
    out = _trace(lambda a, b: turbo.ops.gemm_fp8(a, b, False, True, torch.bfloat16, cfg), a, b)
    assert out.shape == (256, 384) and out.dtype == torch.bfloat16
    assert a.grad.shape == a.shape and b.grad.shape == b.shape


@pytest.mark.parametrize("gran", GRANS)
def test_float8_linear_traces_fullgraph(turbo, gran):
    from primus_turbo.pytorch.modules import Float8Linear

    lin = Float8Linear(512, 256, bias=True, config=_cfg(gran), device="meta", dtype=torch.bfloat16)
    x = _meta(4, 32, 512)
    out = _trace(lin, x)
    assert out.shape == (4, 32, 256) and x.grad.shape == x.shape
    assert lin.weight.grad.shape == lin.weight.shape and lin.bias.grad.shape == lin.bias.shape


@pytest.mark.parametrize("gran", GRANS)
def test_grouped_gemm_fp8_traces_fullgraph(turbo, gran):
    cfg = _cfg(gran)
    a, b = _meta(512, 512), _meta(4, 384, 512)
    lens = torch.empty(4, device="meta", dtype=torch.int64)
    out = _trace(lambda a, b: turbo.ops.grouped_gemm_fp8(a, b, lens, trans_b=True, config=cfg), a, b)
    assert out.shape == (512, 384)
    assert a.grad.shape == a.shape and b.grad.shape == b.shape


def test_fp4_ops_trace_fullgraph(turbo):
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig

    cfg = Float4QuantConfig()
    a, b = _meta(512, 512), _meta(384, 512)
    out = _trace(lambda a, b: turbo.ops.gemm_fp4(a, b, False, True, torch.bfloat16, cfg), a, b)
    assert out.shape == (512, 384) and a.grad.shape == a.shape and b.grad.shape == b.shape
    a, b = _meta(512, 512), _meta(4, 384, 512)
    lens = torch.empty(4, device="meta", dtype=torch.int64)
    out = _trace(lambda a, b: turbo.ops.grouped_gemm_fp4(a, b, lens, trans_b=True, config=cfg), a, b)
    assert out.shape == (512, 384) and a.grad.shape == a.shape and b.grad.shape == b.shape


@pytest.mark.parametrize("kind", ["swiglu", "geglu"])
def test_gated_activation_traces_fullgraph(turbo, kind):
    fn = turbo.ops.swiglu_with_probs if kind == "swiglu" else turbo.ops.geglu_with_probs
    x, p = _meta(300, 512), _meta(300, 1, dtype=torch.float32)
    out = _trace(lambda x, p: fn(x, p, None), x, p)
    assert out.shape == (300, 256) and x.grad.shape == x.shape and p.grad.shape == p.shape


@pytest.mark.parametrize("gran", GRANS + ["mxfp4"])
def test_grouped_linear_traces_fullgraph(turbo, gran):
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig
    from primus_turbo.pytorch.modules import GroupedLinear

    cfg = Float4QuantConfig() if gran == "mxfp4" else _cfg(gran)
    mod = GroupedLinear(4, 512, 512, "meta", dtype=torch.bfloat16, config=cfg)
    x = _meta(1024, 512)
    lens = torch.empty(4, device="meta", dtype=torch.int64)
    out = _trace(mod, x, lens)
    assert out.shape == (1024, 512) and x.grad.shape == x.shape and mod.weight.grad.shape == (4, 512, 512)


def test_mx_dispatcher_meta_shapes_with_shuffled_scales(turbo):
    """Shape functions of the dense MX quantizer operators with shuffle_scale: the scale of every
    matrix is padded to (256, 8) multiples, as the device path returns it."""
    ext = torch.ops.primus_turbo_cpp_extension
    x = torch.empty(3, 136, 160, device="meta", dtype=torch.bfloat16)
    q, s = ext.quantize_mxfp8(x, torch.float8_e4m3fn, 2, 128, False, True, False)
    assert tuple(q.shape) == (3, 136, 256) and tuple(s.shape) == (3, 256, 8)
    q, s = ext.quantize_mxfp8(x, torch.float8_e4m3fn, 2, 128, False, False, False)
    assert tuple(s.shape) == (3, 136, 8)
    rq, rs, cq, cs = ext.quantize_mxfp8_dual(x, torch.float8_e4m3fn, 128, False, False, False, False, True, False)
    assert tuple(rs.shape) == (3, 136, 8) and tuple(cq.shape) == (3, 160, 256) and tuple(cs.shape) == (3, 256, 8)
