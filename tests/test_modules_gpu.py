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


@pytest.mark.parametrize("kind", ["rowwise", "blockwise", "mxfp8", "mxfp4"])
def test_moe_expert_mlp_composition(kind):
    """Two grouped GEMMs around a SwiGLU, the way an MoE expert MLP uses the path (fc1 -> act -> fc2),
    forward and all gradients against the same layer in unquantized bf16 matmuls. Each product alone
    meets the reference's gates (25 dB FP8, 8 dB MXFP4: the grouped GEMM tests); here the
    quantization noise of two layers and of the gradient chain adds up, measured 23-24 dB for FP8:
    the gates are 20 dB (FP8) / 8 dB (MXFP4), 3 dB less for the gradients that pass through both."""
    import numpy as np

    from helpers import bf16_randn, group_lens, to_f32_np
    import primus_turbo.pytorch as turbo
    from oracle import gemm as OG
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig, Float8QuantConfig, Format, ScaleDtype
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G

    E, T, H, F = 4, 2048, 1024, 1536
    lens = group_lens("ragged", E, T, 170)
    gl = torch.from_numpy(lens).cuda()
    if kind == "mxfp4":
        cfg, op, gate = Float4QuantConfig(), turbo.ops.grouped_gemm_fp4, 8.0
    else:
        kw = {"blockwise": dict(granularity=G.BLOCKWISE, block_size=128), "rowwise": dict(granularity=G.ROWWISE),
              "mxfp8": dict(granularity=G.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0)}[kind]
        cfg, op, gate = Float8QuantConfig(format=Format.E4M3, **kw), turbo.ops.grouped_gemm_fp8, 20.0
    x0 = bf16_randn((T, H), seed=171)
    w1_0 = bf16_randn((E, 2 * F, H), seed=172) * (H ** -0.5)
    w2_0 = bf16_randn((E, H, F), seed=173) * (F ** -0.5)
    dy = bf16_randn((T, H), seed=174).cuda()

    def layer(gemm):
        x = x0.clone().cuda().requires_grad_(True)
        w1 = w1_0.to(torch.bfloat16).cuda().requires_grad_(True)
        w2 = w2_0.to(torch.bfloat16).cuda().requires_grad_(True)
        h = gemm(x, w1)
        a, b = h.chunk(2, dim=-1)
        y = gemm(torch.nn.functional.silu(a) * b, w2)
        y.backward(dy)
        return [to_f32_np(t) for t in (y, x.grad, w1.grad, w2.grad)]

    offs = np.concatenate([[0], np.cumsum(lens)])

    def ref_gemm(x, w):  # per-expert bf16 matmul with fp32 accumulation
        return torch.cat([x[offs[g]:offs[g + 1]] @ w[g].t() for g in range(E)], dim=0)

    got = layer(lambda x, w: op(x, w, gl, trans_b=True, config=cfg))
    want = layer(ref_gemm)
    for name, g, w, slack in zip(("out", "dx", "dw1", "dw2"), got, want, (0, 3, 3, 0)):
        snr = OG.snr_db(w, g)
        assert snr > gate - slack, f"{kind} {name}: SNR {snr:.1f} dB"


@pytest.mark.parametrize("kind", ["tensorwise", "rowwise", "blockwise", "mxfp8", "mxfp4"])
@pytest.mark.parametrize("B,M,N,K", [(4, 256, 1024, 2048), (8, 512, 512, 1024)])
@pytest.mark.parametrize("balance", [True, False])
@pytest.mark.parametrize("compiled", [False, True])
def test_grouped_linear(kind, B, M, N, K, balance, compiled):
    """``GroupedLinear`` against one bf16 ``x_g @ W_g^T`` per group: the shapes of the reference's
    tests/pytorch/modules/test_grouped_linear.py:19-60 (B groups of M tokens on average, balanced or
    not, with and without ``torch.compile(fullgraph=True)``), at the SNR gates of the grouped GEMM
    tests (25 dB FP8, 8 dB MXFP4) since the module multiplies in low precision."""
    import numpy as np

    from helpers import group_lens
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig, ScaleDtype
    from primus_turbo.pytorch.modules import GroupedLinear

    if kind == "mxfp4":
        cfg, gate = Float4QuantConfig(), 8.0
    else:
        kw = {"tensorwise": dict(granularity=G.TENSORWISE), "rowwise": dict(granularity=G.ROWWISE),
              "blockwise": dict(granularity=G.BLOCKWISE, block_size=128),
              "mxfp8": dict(granularity=G.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0)}[kind]
        cfg, gate = Float8QuantConfig(format=Format.E4M3, **kw), 25.0
    torch.manual_seed(3)
    torch._dynamo.reset()
    lens = group_lens("balanced" if balance else "ragged", B, B * M, 5)
    gl = torch.from_numpy(lens).cuda()
    mod = GroupedLinear(B, K, N, "cuda", dtype=torch.bfloat16, config=cfg)
    assert tuple(mod.weight.shape) == (B, N, K) and f"group_num={B}" in repr(mod)
    fn = torch.compile(mod, fullgraph=True) if compiled else mod
    x1 = torch.randn((B * M, K), device="cuda", dtype=torch.bfloat16, requires_grad=True)
    x2 = x1.detach().clone().requires_grad_()
    w2 = mod.weight.detach().clone().requires_grad_()
    out1 = fn(x1, gl)
    offs = np.concatenate([[0], np.cumsum(lens)])
    out2 = torch.cat([x2[offs[g]:offs[g + 1]] @ w2[g].t() for g in range(B)], dim=0)
    assert out1.shape == out2.shape and out1.dtype == torch.bfloat16
    go = torch.randn_like(out1)
    out1.backward(go)
    out2.backward(go)
    for name, got, want in (("out", out1, out2), ("dx", x1.grad, x2.grad), ("dw", mod.weight.grad, w2.grad)):
        assert _snr(want, got) > gate, f"{kind} {name}: SNR {_snr(want, got):.1f} dB"


def test_grouped_linear_constructs_like_the_reference_and_needs_a_config_to_run():
    """The reference's constructor signature (no config) constructs; ``forward`` asks for the
    config; assigning one afterwards gives the same result as the constructor keyword."""
    from primus_turbo.pytorch.modules import GroupedLinear

    mod = GroupedLinear(4, 128, 256, "cuda", dtype=torch.bfloat16)
    assert tuple(mod.weight.shape) == (4, 256, 128)
    x = torch.randn(64, 128, device="cuda", dtype=torch.bfloat16)
    lens = torch.tensor([16, 0, 40, 8], dtype=torch.int64, device="cuda")
    with pytest.raises(NotImplementedError, match="Float8QuantConfig"):
        mod(x, lens)
    cfg = Float8QuantConfig(granularity=G.BLOCKWISE, block_size=128)
    mod.config = cfg
    y = mod(x, lens)
    mod2 = GroupedLinear(4, 128, 256, "cuda", dtype=torch.bfloat16, config=cfg)
    with torch.no_grad():
        mod2.weight.copy_(mod.weight)
    assert torch.equal(y, mod2(x, lens))


@pytest.mark.parametrize("kind", ["rowwise", "blockwise", "mxfp8"])
def test_moe_layer_permute_experts_unpermute(kind):
    """A whole MoE expert layer on the path: ``moe_permute`` (top-k routing, groups padded to 32 rows)
    -> grouped fc1 -> ``swiglu_with_probs`` -> grouped fc2 -> ``moe_unpermute``, forward and all
    gradients, against the same layer computed token by token in fp32 from the bf16 values. The
    permute's ``tokens_per_expert`` is the group-length tensor of the grouped GEMMs as it stands (no
    host round trip). Gates as in the two-GEMM composition above (20 dB, 17 dB for gradients through
    both products); the gradient of the router probabilities passes through one product: 20 dB."""
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import ScaleDtype

    T, E, K, H, F, pad = 512, 8, 2, 512, 768, 32
    kw = {"blockwise": dict(granularity=G.BLOCKWISE, block_size=128), "rowwise": dict(granularity=G.ROWWISE),
          "mxfp8": dict(granularity=G.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0)}[kind]
    cfg = Float8QuantConfig(format=Format.E4M3, **kw)
    g = torch.Generator().manual_seed(77)
    x0 = torch.randn(T, H, generator=g).to(torch.bfloat16)
    w1_0 = (torch.randn(E, 2 * F, H, generator=g) * H ** -0.5).to(torch.bfloat16)
    w2_0 = (torch.randn(E, H, F, generator=g) * F ** -0.5).to(torch.bfloat16)
    p0 = torch.rand(T, K, generator=g) + 0.25
    topk = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    dy = torch.randn(T, H, generator=g).to(torch.bfloat16).cuda()

    def leaves(dtype):
        return [t.clone().to(dtype).cuda().requires_grad_(True) for t in (x0, w1_0, w2_0, p0)]

    x, w1, w2, p = leaves(torch.bfloat16)
    p = p0.clone().cuda().requires_grad_(True)
    rows = T * K + E * pad  # an upper bound keeps the op free of a host read-back
    px, rmap, tpe, overflow, nd, _, pp = turbo.ops.moe_permute(
        x, topk.cuda(), num_local_experts=E, num_topk=K, pad_multiple=pad, num_permuted_tokens=rows, probs=p,
        probs_layout="topk")
    assert px.shape[0] == rows and int(overflow.item()) == 0
    used = int(tpe.sum().item())
    px, pp = px[:used], pp[:used]  # the rows the experts own; the tail of the bound is unused
    h = turbo.ops.grouped_gemm_fp8(px, w1, tpe, trans_b=True, config=cfg)
    a = turbo.ops.swiglu_with_probs(h, pp.unsqueeze(-1), None)
    y = turbo.ops.grouped_gemm_fp8(a, w2, tpe, trans_b=True, config=cfg)
    y = torch.cat([y, y.new_zeros(rows - used, H)])
    out, _ = turbo.ops.moe_unpermute(y, rmap, nd, restore_shape=x.shape, num_local_experts=E, pad_multiple=pad)
    out.backward(dy)

    xr, w1r, w2r, pr = leaves(torch.float32)
    ref = torch.zeros(T, H, device="cuda")
    for k in range(K):
        e = topk[:, k].cuda()
        hk = torch.einsum("th,tfh->tf", xr, w1r[e])
        ak = torch.nn.functional.silu(hk[:, :F]) * hk[:, F:] * pr[:, k:k + 1]
        ref = ref + torch.einsum("tf,thf->th", ak, w2r[e])
    ref.backward(dy.float())
    for name, got, want, gate in (("out", out, ref, 20.0), ("dx", x.grad, xr.grad, 17.0), ("dw1", w1.grad, w1r.grad, 17.0),
                                  ("dw2", w2.grad, w2r.grad, 20.0), ("dprobs", p.grad, pr.grad, 20.0)):
        assert _snr(want, got) > gate, f"{kind} {name}: SNR {_snr(want, got):.1f} dB"
