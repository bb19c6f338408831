"""Results under ``torch.compile`` equal the eager results bit for bit: the compiled graph calls
the same HIP kernels through the registered operators. Mirrors the ``enable_torch_compile`` leg
of the reference's FP8 linear test (tests/pytorch/modules/test_linear_fp8.py:33-70, compiled with
``fullgraph=False``) and widens it to ``fullgraph=True`` over every op family."""

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo
    import primus_turbo.pytorch as turbo


def _cfg(name):
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, ScaleDtype, ScalingGranularity as G

    return {
        "tensorwise": lambda: Float8QuantConfig(granularity=G.TENSORWISE),
        "rowwise": lambda: Float8QuantConfig(granularity=G.ROWWISE),
        "blockwise": lambda: Float8QuantConfig(granularity=G.BLOCKWISE, block_size=128),
        "mx": lambda: Float8QuantConfig(granularity=G.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0),
    }[name]()


def _rand(*shape, dtype=torch.bfloat16, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype).cuda().requires_grad_(True)


def _run(fn, args, params=()):
    leaves = list(args) + list(params)
    for t in leaves:
        t.grad = None
    out = fn(*args)
    out.float().sum().backward()
    torch.cuda.synchronize()
    return out.detach().clone(), [t.grad.detach().clone() for t in leaves if t.requires_grad]


def _same_as_eager(fn, args, fullgraph, params=()):
    torch._dynamo.reset()
    out_e, grads_e = _run(fn, args, params)
    out_c, grads_c = _run(torch.compile(fn, fullgraph=fullgraph), args, params)
    assert torch.equal(out_e, out_c), "forward differs under torch.compile"
    assert len(grads_e) == len(grads_c)
    for i, (e, c) in enumerate(zip(grads_e, grads_c)):
        assert torch.equal(e, c), f"gradient {i} differs under torch.compile"


GRANS = ["tensorwise", "rowwise", "blockwise", "mx"]


@pytest.mark.parametrize("gran", GRANS)
@pytest.mark.parametrize("fullgraph", [False, True])
def test_float8_linear_compiled(gran, fullgraph):
    from primus_turbo.pytorch.modules import Float8Linear

    torch.manual_seed(1)
    lin = Float8Linear(512, 256, bias=True, config=_cfg(gran), device="cuda", dtype=torch.bfloat16)
    x = _rand(4, 32, 512)
    _same_as_eager(lin, (x,), fullgraph, params=list(lin.parameters()))


@pytest.mark.parametrize("gran", GRANS)
def test_gemm_fp8_compiled(gran):
    cfg = _cfg(gran)
    a, b = _rand(256, 512), _rand(384, 512, seed=1)
    _same_as_eager(lambda a, b: turbo.ops.gemm_fp8(a, b, False, True, torch.bfloat16, cfg), (a, b), True)


@pytest.mark.parametrize("gran", GRANS)
def test_grouped_gemm_fp8_compiled(gran):
    cfg = _cfg(gran)
    a, b = _rand(512, 512), _rand(4, 512, 512, seed=1)  # the MX kernels want every reduction length >= 512
    lens = torch.tensor([128, 96, 160, 128], dtype=torch.int64).cuda()
    _same_as_eager(lambda a, b: turbo.ops.grouped_gemm_fp8(a, b, lens, trans_b=True, config=cfg), (a, b), True)


def test_fp4_ops_compiled():
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig

    cfg = Float4QuantConfig()  # deterministic rounding: stochastic rounding draws a fresh seed per call
    a, b = _rand(512, 512), _rand(384, 512, seed=1)
    _same_as_eager(lambda a, b: turbo.ops.gemm_fp4(a, b, False, True, torch.bfloat16, cfg), (a, b), True)
    a, b = _rand(512, 512), _rand(4, 384, 512, seed=1)
    lens = torch.tensor([128, 96, 160, 128], dtype=torch.int64).cuda()
    _same_as_eager(lambda a, b: turbo.ops.grouped_gemm_fp4(a, b, lens, trans_b=True, config=cfg), (a, b), True)


@pytest.mark.parametrize("kind", ["swiglu", "geglu"])
def test_gated_activation_compiled(kind):
    fn = turbo.ops.swiglu_with_probs if kind == "swiglu" else turbo.ops.geglu_with_probs
    x = _rand(300, 512)
    p = torch.rand(300, 1, generator=torch.Generator().manual_seed(2)).cuda().requires_grad_(True)
    _same_as_eager(lambda x, p: fn(x, p, None), (x, p), True)


@pytest.mark.parametrize("gran", GRANS)
def test_float8_linear_max_autotune(gran):
    """``mode="max-autotune"``, the setting of the reference's test: Inductor then runs the graph
    through CUDA-graph trees (warm-up, capture, replays), so the ops must be capturable and must keep
    nothing alive in the graph's memory pool. Fresh inputs on every call; each call equals eager."""
    from primus_turbo.pytorch.modules import Float8Linear

    torch._dynamo.reset()
    torch.manual_seed(2)
    lin = Float8Linear(512, 256, bias=True, config=_cfg(gran), device="cuda", dtype=torch.bfloat16)
    compiled = torch.compile(lin, fullgraph=False, mode="max-autotune")
    for it in range(4):
        x = _rand(128, 512, seed=10 + it)
        out_e, grads_e = _run(lin, (x,), list(lin.parameters()))
        out_c, grads_c = _run(compiled, (x,), list(lin.parameters()))
        assert torch.equal(out_e, out_c), f"call {it}: forward differs"
        for e, c in zip(grads_e, grads_c):
            assert torch.equal(e, c), f"call {it}: a gradient differs"
