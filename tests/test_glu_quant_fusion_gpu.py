"""The gated activation fused into the grouped quantizers (blockwise FP8, MXFP8, MXFP4), and the
fused activation -> grouped GEMM operations built on them.

Oracle = composition: ``oracle.activation`` (tolerance: floating point) -> the 16-bit rounding the
stand-alone activation kernel stores -> ``oracle.quantize.fp8_blockwise_segment_m_row_col`` (bit-exact
on that stored activation). The fused kernel has to give, bit for bit, what the two steps of this
library give one after the other; the two steps are each checked against their oracles here too."""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, bits_np, codes_np, group_lens, to_f32_np
from oracle import activation as OA
from oracle import quantize as Q

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, qi, G, Float8QuantConfig, ScalingRecipe
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, ScalingRecipe
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi


def _inputs(kind, G_, M, H, dtype, seed, masked):
    lens = group_lens(kind, G_, M, seed)
    gl = torch.from_numpy(lens).cuda()
    offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)
    x = bf16_randn((M, 2 * H), seed=seed + 1, scale=1.5, dtype=dtype).cuda()
    g = torch.Generator().manual_seed(seed + 2)
    probs = torch.rand(M, generator=g, dtype=torch.float32).cuda()
    mask = None
    if masked:
        mask = (torch.rand(M, generator=g) > 0.2).to(torch.int64).cuda()
    return lens, gl, offs, x, probs, mask


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind,G_,M,H,masked", [("balanced", 4, 1024, 512, False), ("ragged", 8, 3000, 384, True),
                                                ("zeros", 8, 2048, 256, False), ("ragged", 3, 77, 100, True),
                                                ("zipf", 32, 8192, 2048, True)])
def test_fused_quantizer_equals_the_two_steps_and_the_oracle(kind, G_, M, H, masked, dtype, act):
    lens, gl, offs, x, probs, mask = _inputs(kind, G_, M, H, dtype, 81, masked)
    f8 = torch.float8_e4m3fn
    two = turbo.ops.swiglu_with_probs if act == "silu" else turbo.ops.geglu_with_probs
    y = two(x, probs, mask)  # the stored activation of the two-step path
    # activation against its oracle (float64 formula; one rounding of the 16-bit format + fp32 evaluation)
    ref = OA.glu_with_probs(to_f32_np(x), probs.cpu().numpy(), act, None if mask is None else mask.cpu().numpy())
    tol = 2.0 ** (-8 if dtype == torch.bfloat16 else -10)
    assert np.all(np.abs(to_f32_np(y) - ref) <= tol * np.abs(ref) + 1e-6)

    for transposed in (False, True):
        step2 = qi.quant_fp8_blockwise_segment_m_row_col_t_impl if transposed else qi.quant_fp8_blockwise_segment_m_row_col_impl
        want = step2(y, f8, 128, gl, offs)
        got = qi.glu_quant_fp8_blockwise_segment_m_row_col_impl(x, probs, mask, act, f8, 128, gl, offs, transposed)
        torch.cuda.synchronize()
        w = int(want[5][-1].item())  # rows of the padded column output that exist
        assert torch.equal(got[0].view(torch.uint8), want[0].view(torch.uint8)), "row codes"
        assert torch.equal(got[2], want[2]), "row scales"
        if transposed:
            assert torch.equal(got[1].view(torch.uint8)[:, :w], want[1].view(torch.uint8)[:, :w]), "transposed column codes"
        else:
            assert torch.equal(got[1].view(torch.uint8)[:w], want[1].view(torch.uint8)[:w]), "column codes"
        assert torch.equal(got[3][: w // 128], want[3][: w // 128]), "column scales"
        assert torch.equal(got[4], want[4]) and torch.equal(got[5], want[5])

    # the quantizer oracle on the stored activation: bit-exact
    o = Q.fp8_blockwise_segment_m_row_col(to_f32_np(y), lens, "e4m3")
    got = qi.glu_quant_fp8_blockwise_segment_m_row_col_impl(x, probs, mask, act, f8, 128, gl, offs, False)
    wr = o["written_rows"]
    assert np.array_equal(codes_np(got[0]), o["row"])
    assert np.array_equal(bits_np(got[2]), o["row_scale"].view(np.uint32))
    assert np.array_equal(codes_np(got[1])[:wr], o["col"][:wr])
    assert np.array_equal(bits_np(got[3])[: wr // 128], o["col_scale"].view(np.uint32)[: wr // 128])


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("trans_b", [True, False])
def test_fused_activation_grouped_gemm_equals_the_two_step_layer(act, trans_b):
    """fc2 of an expert MLP: ``glu_grouped_gemm_fp8`` against ``grouped_gemm_fp8(swiglu_with_probs(...))``,
    output and all three gradients, bit for bit."""
    G_, M, H, N = 8, 2048, 512, 768
    lens, gl, offs, x, probs, mask = _inputs("zipf", G_, M, H, torch.bfloat16, 91, True)
    w = bf16_randn((G_, N, H) if trans_b else (G_, H, N), seed=95, scale=0.05).cuda()
    dy = bf16_randn((M, N), seed=96).cuda()
    cfg = Float8QuantConfig(granularity=G.BLOCKWISE, block_size=128)

    def run(fused):
        xx, pp, ww = x.clone().requires_grad_(True), probs.clone().requires_grad_(True), w.clone().requires_grad_(True)
        if fused:
            out = turbo.ops.glu_grouped_gemm_fp8(xx, pp, ww, gl, offs, trans_b=trans_b, config=cfg, row_mask=mask, act_type=act)
        else:
            two = turbo.ops.swiglu_with_probs if act == "silu" else turbo.ops.geglu_with_probs
            out = turbo.ops.grouped_gemm_fp8(two(xx, pp, mask), ww, gl, offs, trans_b=trans_b, config=cfg)
        out.backward(dy)
        return out.detach(), xx.grad, pp.grad, ww.grad

    a, b = run(True), run(False)
    for name, u, v in zip(("out", "grad_x", "grad_probs", "grad_w"), a, b):
        assert torch.equal(u, v), name
    # inference (no gradient needed): the untransposed column output path
    with torch.no_grad():
        out = turbo.ops.glu_grouped_gemm_fp8(x, probs, w, gl, offs, trans_b=trans_b, config=cfg, row_mask=mask, act_type=act)
    assert torch.equal(out, a[0])


def test_fused_activation_grouped_gemm_mixed_dtypes():
    """fp16 activations, a bf16 weight and an explicit out_dtype: the activation gradient comes
    back in the activation's type and the weight gradient in out_dtype."""
    G_, M, H, N = 4, 1024, 256, 384
    lens, gl, offs, x, probs, mask = _inputs("ragged", G_, M, H, torch.float16, 97, False)
    w = bf16_randn((G_, N, H), seed=98, scale=0.05).cuda()
    dy = bf16_randn((M, N), seed=99).cuda()
    cfg = Float8QuantConfig(granularity=G.BLOCKWISE, block_size=128)

    def run(fused):
        xx, pp, ww = x.clone().requires_grad_(True), probs.clone().requires_grad_(True), w.clone().requires_grad_(True)
        if fused:
            out = turbo.ops.glu_grouped_gemm_fp8(xx, pp, ww, gl, offs, trans_b=True, config=cfg, act_type="silu",
                                                 out_dtype=torch.bfloat16)
        else:
            out = turbo.ops.grouped_gemm_fp8(turbo.ops.swiglu_with_probs(xx, pp, None), ww, gl, offs, trans_b=True,
                                             out_dtype=torch.bfloat16, config=cfg)
        assert out.dtype == torch.bfloat16
        out.backward(dy)
        return out.detach(), xx.grad, pp.grad, ww.grad

    a, b = run(True), run(False)
    assert a[1].dtype == torch.float16 and a[3].dtype == torch.bfloat16
    for name, u, v in zip(("out", "grad_x", "grad_probs", "grad_w"), a, b):
        assert u.dtype == v.dtype, name
    assert torch.equal(a[0], b[0]) and torch.equal(a[3], b[3]), "output and weight gradient: same GEMMs, same types"
    # the two-step form rounds the activation gradient to out_dtype (bf16) before autograd casts it to
    # fp16; the fused form writes fp16 from the fp32 sums directly: equal up to that bf16 rounding
    for u, v in ((a[1], b[1]), (a[2], b[2])):
        assert (u.float() - v.float()).norm() <= 2.0 ** -7 * v.float().norm()


# ---- the grouped MX quantizers (MXFP8 / MXFP4) with the gated activation applied on load ----
MX_CASES = [("balanced", 4, 1024, 512, False), ("ragged", 8, 3000, 384, True), ("zeros", 8, 2048, 256, False),
            ("ragged", 3, 77, 96, True), ("zipf", 32, 8192, 2048, True)]


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
@pytest.mark.parametrize("kind,G_,M,H,masked", MX_CASES)
def test_fused_mx_quantizer_equals_the_two_steps_and_the_oracle(kind, G_, M, H, masked, fmt, dtype, act):
    lens, gl, offs, x, probs, mask = _inputs(kind, G_, M, H, dtype, 181, masked)
    fp4 = fmt == "e2m1"
    qdt = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2, "e2m1": torch.float4_e2m1fn_x2}[fmt]
    two = turbo.ops.swiglu_with_probs if act == "silu" else turbo.ops.geglu_with_probs
    y = two(x, probs, mask)  # the stored activation of the two-step path (checked against its oracle above)
    col_flags = 2 if fp4 else 0  # MXFP4's wgrad operand is Hadamard-transformed along the tokens
    got = qi.glu_grouped_quantize_mx_impl(x, probs, mask, act, qdt, gl, offs, True, col_flags)
    if fp4:
        want = qi.grouped_quantize_mxfp4_impl(y, qdt, None, 32, gl, offs, with_trans=True, scaling_recipe=ScalingRecipe(),
                                              scaling_recipe_for_trans=ScalingRecipe(use_rht=True))
    else:
        want = qi.grouped_quantize_mxfp8_impl(y, qdt, None, 32, gl, offs, with_trans=True)
    torch.cuda.synchronize()
    o = Q.mx_grouped_quant(to_f32_np(y), lens, fmt, row_align=1 if fp4 else 32, col_align=256 if fp4 else 128,
                           col_rht=fp4)
    mr, mc = int(o["row_offs"][-1]), int(o["col_offs"][-1])
    pack = 2 if fp4 else 1
    # bit for bit the two-step result ...
    assert np.array_equal(codes_np(got[0])[:mr], codes_np(want[0])[:mr]), "row codes"
    assert np.array_equal(codes_np(got[1])[:mr], codes_np(want[1])[:mr]), "row scales"
    assert np.array_equal(codes_np(got[2])[:, : mc // pack], codes_np(want[2])[:, : mc // pack]), "column codes"
    assert np.array_equal(codes_np(got[3])[:, : mc // 32], codes_np(want[3])[:, : mc // 32]), "column scales"
    assert torch.equal(got[6], want[6]) and torch.equal(got[7], want[7])
    if not fp4:
        assert torch.equal(got[4], want[4]) and torch.equal(got[5], want[5])
    # ... and the quantizer oracle on the stored activation
    assert np.array_equal(codes_np(got[0])[:mr], o["row"]) and np.array_equal(codes_np(got[1])[:mr], o["row_scale"])
    assert np.array_equal(codes_np(got[2])[:, : mc // pack], o["col"])
    assert np.array_equal(codes_np(got[3])[:, : mc // 32], o["col_scale"])
    # rows only (inference): the same row pair
    r = qi.glu_grouped_quantize_mx_impl(x, probs, mask, act, qdt, gl, offs, False)
    assert np.array_equal(codes_np(r[0])[:mr], o["row"]) and np.array_equal(codes_np(r[1])[:mr], o["row_scale"])
    assert r[2].numel() == 0 and r[3].numel() == 0


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("fp4", [False, True])
def test_fused_activation_grouped_mx_gemm_equals_the_two_step_layer(act, fp4):
    """fc2 of an expert MLP on MXFP8 / MXFP4 operands: the fused operation against
    ``grouped_gemm_fp8/fp4(swiglu_with_probs(...))``, output and all three gradients, bit for bit."""
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig, ScaleDtype

    G_, M, H, N = 8, 2048, 512, 768
    lens, gl, offs, x, probs, mask = _inputs("zipf", G_, M, H, torch.bfloat16, 191, True)
    w = bf16_randn((G_, N, H), seed=195, scale=0.05).cuda()
    dy = bf16_randn((M, N), seed=196).cuda()
    if fp4:
        cfg = Float4QuantConfig()
        fused_op, plain_op = turbo.ops.glu_grouped_gemm_fp4, turbo.ops.grouped_gemm_fp4
    else:
        cfg = Float8QuantConfig(granularity=G.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0)
        fused_op, plain_op = turbo.ops.glu_grouped_gemm_fp8, turbo.ops.grouped_gemm_fp8

    def run(fused):
        xx, pp, ww = x.clone().requires_grad_(True), probs.clone().requires_grad_(True), w.clone().requires_grad_(True)
        if fused:
            out = fused_op(xx, pp, ww, gl, offs, config=cfg, row_mask=mask, act_type=act)
        else:
            two = turbo.ops.swiglu_with_probs if act == "silu" else turbo.ops.geglu_with_probs
            out = plain_op(two(xx, pp, mask), ww, gl, offs, config=cfg)
        out.backward(dy)
        return out.detach(), xx.grad, pp.grad, ww.grad

    a, b = run(True), run(False)
    for name, u, v in zip(("out", "grad_x", "grad_probs", "grad_w"), a, b):
        assert torch.equal(u, v), name
    with torch.no_grad():
        out = fused_op(x, probs, w, gl, offs, config=cfg, row_mask=mask, act_type=act)
    assert torch.equal(out, a[0])
