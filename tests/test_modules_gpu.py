"""``Float8Linear`` against ``torch.nn.Linear``: forward, dgrad and wgrad at the reference's SNR
gate (tests/pytorch/modules/test_linear_fp8.py of the reference: 20 dB), bias gradient exact to the
dtype's tolerance; conversion in place and into a copy."""

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global Float8Linear, Float8QuantConfig, Format, G
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, Format
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.modules import Float8Linear


def _snr(ref, got):
    ref, got = ref.detach().float(), got.detach().float()
    return float(10 * torch.log10(ref.pow(2).sum() / (ref - got).pow(2).sum().clamp_min(1e-30)))


def _configs():
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, Format
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G

    out = []
    for gran, kw in ((G.TENSORWISE, {}), (G.ROWWISE, {}), (G.BLOCKWISE, {"block_size": 128})):
        for fmt in (Format.E4M3, Format.E5M2, Format.HYBRID):
            if fmt == Format.HYBRID and gran != G.TENSORWISE:
                continue
            out.append((gran, kw, fmt))
    return out


@pytest.mark.parametrize("case", range(7))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K", [(128, 256, 512), (4096, 256, 2048), (96, 4096, 512)])
@pytest.mark.parametrize("bias", [True, False])
def test_float8linear_matches_linear(case, dtype, M, N, K, bias):
    gran, kw, fmt = _configs()[case]
    cfg = Float8QuantConfig(granularity=gran, format=fmt, **kw)
    torch.manual_seed(17)
    x1 = torch.randn((M, K), dtype=dtype, device="cuda", requires_grad=True)
    x2 = x1.detach().clone().requires_grad_()
    ref = torch.nn.Linear(K, N, bias=bias).to("cuda", dtype=dtype)
    out_ref = ref(x1)
    g = torch.randn_like(out_ref)
    out_ref.backward(g)
    xg_ref, wg_ref = x1.grad.clone(), ref.weight.grad.clone()
    bg_ref = ref.bias.grad.clone() if bias else None
    ref.weight.grad = None
    if bias:
        ref.bias.grad = None

    mod = Float8Linear.from_float(ref, cfg)
    assert isinstance(mod, Float8Linear) and mod is ref and "config=" in repr(mod)
    out = mod(x2)
    assert out.shape == (M, N) and out.dtype == dtype
    out.backward(g)
    assert _snr(out_ref, out) > 20
    assert _snr(xg_ref, x2.grad) > 20
    assert _snr(wg_ref, mod.weight.grad) > 20
    if bias:
        tol = dict(rtol=1.6e-2, atol=1e-5) if dtype == torch.bfloat16 else dict(rtol=1e-3, atol=1e-5)
        torch.testing.assert_close(mod.bias.grad, bg_ref, **tol)


def test_float8linear_copy_conversion_and_batched_input():
    torch.manual_seed(18)
    lin = torch.nn.Linear(512, 384, bias=True).to("cuda", dtype=torch.bfloat16)
    mod = Float8Linear.from_float(lin, None, inplace=False)
    assert mod is not lin and type(lin) is torch.nn.Linear
    assert mod.config.granularity == G.TENSORWISE
    assert torch.equal(mod.weight, lin.weight) and torch.equal(mod.bias, lin.bias)
    x = torch.randn((4, 33, 512), dtype=torch.bfloat16, device="cuda")
    y = mod(x)
    assert y.shape == (4, 33, 384)
    assert _snr(lin(x), y) > 20
    direct = Float8Linear(512, 384, bias=False, config=Float8QuantConfig(granularity=G.ROWWISE), device="cuda",
                          dtype=torch.bfloat16)
    assert direct(x).shape == (4, 33, 384)
