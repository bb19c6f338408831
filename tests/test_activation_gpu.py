"""GPU parity of ``swiglu_with_probs`` / ``geglu_with_probs`` (the reference's
tests/pytorch/ops/test_activation.py:60-160 cases: token counts 1 ... 8192 incl. 2025, hidden 128 /
256 / 2048, bf16 / fp16, with and without a row mask) against the float64 oracle. Tolerance:
floating point, so one rounding of the output format (2^-8 relative for bf16, 2^-11 for fp16) plus
the fp32 evaluation error of exp / erf (<= 4 ulp): |got - ref| <= 1.01 * 2^-8 (2^-11) * |ref| +
1e-6 * max|ref| for the 16-bit outputs, 2e-5 relative to the row's abs-sum for the fp32 row sums."""

import numpy as np
import pytest
import torch

from helpers import to_f32_np
from oracle import activation as A

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo
    import primus_turbo.pytorch as turbo


def _close16(got, ref, dtype, what):
    rel = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11
    tol = 1.01 * rel * np.abs(ref) + 1e-6 * np.abs(ref).max() + 1e-30
    bad = np.abs(got.astype(np.float64) - ref) > tol
    assert not bad.any(), f"{what}: {bad.sum()} of {bad.size} outside tolerance, worst {np.abs(got - ref).max():.3e}"


@pytest.mark.parametrize("kind", ["silu", "gelu"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("tokens,hidden", [(1, 128), (128, 256), (2025, 2048), (8192, 128), (300, 100), (64, 7168)])
@pytest.mark.parametrize("masked", [False, True])
def test_glu_with_probs(kind, dtype, tokens, hidden, masked):
    g = torch.Generator().manual_seed(7)
    x = torch.randn(tokens, 2 * hidden, generator=g).to(dtype)
    probs = torch.rand(tokens, generator=g, dtype=torch.float32)
    go = torch.randn(tokens, hidden, generator=g).to(dtype)
    mask = None
    if masked:
        mask = torch.zeros(tokens, dtype=torch.int64)
        mask[: max(1, (3 * tokens) // 4)] = 1
    xd = x.cuda().requires_grad_(True)
    pd = probs.cuda().requires_grad_(True)
    fn = turbo.ops.swiglu_with_probs if kind == "silu" else turbo.ops.geglu_with_probs
    out = fn(xd, pd, None if mask is None else mask.cuda())
    assert out.shape == (tokens, hidden) and out.dtype == dtype
    out.backward(go.cuda())
    torch.cuda.synchronize()
    m = None if mask is None else mask.numpy()
    ref = A.glu_with_probs(to_f32_np(x), probs.numpy(), kind, m)
    _close16(to_f32_np(out), ref, dtype, "forward")
    gx, gp = A.glu_with_probs_grad(to_f32_np(go), to_f32_np(x), probs.numpy(), kind, m)
    _close16(to_f32_np(xd.grad), gx, dtype, "grad_x")
    H = hidden
    xf, gof = to_f32_np(x).astype(np.float64), to_f32_np(go).astype(np.float64)
    row_abs = np.abs(gof * A.act(xf[:, :H], kind) * xf[:, H:]).sum(axis=1)
    assert np.all(np.abs(pd.grad.cpu().numpy().astype(np.float64) - gp) <= 2e-5 * row_abs + 1e-30), "grad_probs"
    if masked:
        dead = mask.numpy() == 0
        assert not to_f32_np(out)[dead].any() and not to_f32_np(xd.grad)[dead].any()


def test_glu_shapes_and_errors():
    x = torch.randn(2, 8, 64, dtype=torch.bfloat16, device="cuda", requires_grad=True)
    probs = torch.rand(2, 8, dtype=torch.float32, device="cuda", requires_grad=True)
    out = turbo.ops.swiglu_with_probs(x, probs)
    assert out.shape == (16, 32)
    out.sum().backward()
    assert x.grad.shape == x.shape and probs.grad.shape == probs.shape
    with pytest.raises(AssertionError):
        turbo.ops.swiglu_with_probs(x, probs.half())
    with pytest.raises(AssertionError):
        turbo.ops.swiglu_with_probs(x, probs, torch.ones(16, dtype=torch.int32, device="cuda"))
    with pytest.raises(RuntimeError):
        turbo.ops.swiglu_with_probs(x.float(), probs)
