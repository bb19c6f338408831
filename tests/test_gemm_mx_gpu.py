"""GPU parity of the MX-scaled GEMMs (MXFP8, MXFP4): the matrix core applies the E8M0 block
scales, so the checks here pin the scale-byte to lane mapping as well as the product.

Gate: against the fp32 matmul of the de-quantized operands, max |err| / max |ref| <= 1e-2 and
cosine >= 0.9999; the autograd ops are held to the reference's SNR gates against the
unquantized computation (tests/pytorch/ops/test_gemm_fp8.py: 25 dB E4M3 / 20 dB E5M2,
tests/pytorch/ops/test_gemm_fp4.py: 10 dB).
"""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, codes_np, gemm_gate, to_f32_np
from oracle import gemm as OG
from oracle import quantize as Q

pytestmark = pytest.mark.gpu

FP4 = getattr(torch, "float4_e2m1fn_x2", None)
MAX_REL = 1e-2
MIN_COS = 0.9999


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, Float8QuantConfig, Float4QuantConfig, Format, ScaleDtype, ScalingRecipe, qi, gi, g4
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig, Float8QuantConfig, Format, ScaleDtype, ScalingRecipe
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.kernels.gemm import gemm_fp4_impl as g4
    from primus_turbo.pytorch.kernels.gemm import gemm_fp8_impl as gi
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi


def _gate(ref, got, what=""):
    return gemm_gate(ref, got, what)


SHAPES = [(256, 256, 384), (512, 384, 1024), (130, 70, 160), (64, 96, 96), (1024, 2048, 512), (300, 260, 2080)]


@pytest.mark.parametrize("M,N,K", SHAPES)
@pytest.mark.parametrize("fa,fb", [("e4m3", "e4m3"), ("e5m2", "e4m3"), ("e4m3", "e5m2")])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_mxfp8_gemm_matches_dequantized_matmul(M, N, K, fa, fb, out_dtype):
    if out_dtype == torch.float32 and (fa, fb) != ("e4m3", "e4m3"):
        pytest.skip("fp32 output is covered once per shape")
    dts = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}
    a = bf16_randn((M, K), seed=60, outlier_frac=0.002).cuda()
    b = bf16_randn((N, K), seed=61).cuda()
    aq, as_ = qi.quantize_mxfp8_impl(a, dts[fa], 1, 32)
    bq, bs = qi.quantize_mxfp8_impl(b, dts[fb], 1, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))
    out = gi.gemm_fp8_impl(aq, as_, False, bq, bs, True, out_dtype, False, G.MX_BLOCKWISE.value, 0)
    out_t = gi.gemm_fp8_impl(aq, as_, False, bq, bs, True, out_dtype, True, G.MX_BLOCKWISE.value, 0)
    torch.cuda.synchronize()
    ref = OG.gemm_dequantized(Q.mx_dequant(codes_np(aq), codes_np(as_), fa), Q.mx_dequant(codes_np(bq), codes_np(bs), fb))
    _gate(ref, to_f32_np(out), f"mxfp8 {fa}x{fb} {M}x{N}x{K}")
    assert torch.equal(out_t, out.t().contiguous())


@pytest.mark.skipif(FP4 is None, reason="torch has no float4_e2m1fn_x2")
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_mxfp4_gemm_matches_dequantized_matmul(M, N, K):
    a = bf16_randn((M, K), seed=62, outlier_frac=0.002).cuda()
    b = bf16_randn((N, K), seed=63).cuda()
    aq, as_ = qi.quantize_mxfp4_impl(a, FP4, 1, 32)
    bq, bs = qi.quantize_mxfp4_impl(b, FP4, 1, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))
    out = g4.gemm_fp4_impl(aq, as_, False, bq, bs, True, torch.float32, False, G.MX_BLOCKWISE.value, 0)
    torch.cuda.synchronize()
    ref = OG.gemm_dequantized(Q.mx_dequant(codes_np(aq), codes_np(as_), "e2m1"), Q.mx_dequant(codes_np(bq), codes_np(bs), "e2m1"))
    _gate(ref, to_f32_np(out), f"mxfp4 {M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", SHAPES + [(2048, 2304, 4224)])
@pytest.mark.parametrize("fmt", ["e4m3", "e5m2", "e2m1"])
def test_mx_gemm_eight_wavefront_tile(M, N, K, fmt):
    """tile_cfg 4 (256 x 256 tile, eight wavefronts, gemm_mx8.h) against the oracle and against the
    automatic configuration: the same products added in the same order, so the bits are the same.
    Exact-integer operands on the same path in the next test."""
    if fmt == "e2m1" and FP4 is None:
        pytest.skip("torch has no float4_e2m1fn_x2")
    a = bf16_randn((M, K), seed=71, outlier_frac=0.002).cuda()
    b = bf16_randn((N, K), seed=72).cuda()
    if fmt == "e2m1":
        aq, as_ = qi.quantize_mxfp4_impl(a, FP4, 1, 32)
        bq, bs = qi.quantize_mxfp4_impl(b, FP4, 1, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))
        run = lambda: g4.gemm_fp4_impl(aq, as_, False, bq, bs, True, torch.float32, False, G.MX_BLOCKWISE.value, 0)  # noqa: E731
    else:
        dt = torch.float8_e4m3fn if fmt == "e4m3" else torch.float8_e5m2
        aq, as_ = qi.quantize_mxfp8_impl(a, dt, 1, 32)
        bq, bs = qi.quantize_mxfp8_impl(b, torch.float8_e4m3fn, 1, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))
        run = lambda: gi.gemm_fp8_impl(aq, as_, False, bq, bs, True, torch.bfloat16, False, G.MX_BLOCKWISE.value, 0)  # noqa: E731
    auto = run()
    gi.TILE_CFG = 4
    try:
        got = run()
    finally:
        gi.TILE_CFG = 0
    torch.cuda.synchronize()
    assert torch.equal(got, auto), "tile configurations differ"
    ref = OG.gemm_dequantized(Q.mx_dequant(codes_np(aq), codes_np(as_), fmt),
                              Q.mx_dequant(codes_np(bq), codes_np(bs), "e2m1" if fmt == "e2m1" else "e4m3"))
    _gate(ref, to_f32_np(got), f"mx8 {fmt} {M}x{N}x{K}")


def test_mx_gemm_without_workspace_reads_scales_in_place():
    """Whole-slab operand rows need no copy: pt_gemm_mx then works with no workspace at all (the
    word-major scale copy of large problems is an option that a sufficient workspace buys), and
    gives the same bits either way."""
    from primus_turbo import _native as N

    lib = N.lib()
    M, Nn, K = 1024, 1280, 2048
    a = bf16_randn((M, K), seed=73, outlier_frac=0.002).cuda()
    b = bf16_randn((Nn, K), seed=74).cuda()
    aq, as_ = qi.quantize_mxfp8_impl(a, torch.float8_e4m3fn, 1, 32)
    bq, bs = qi.quantize_mxfp8_impl(b, torch.float8_e4m3fn, 1, 32)
    want = lib.pt_gemm_mx_workspace_bytes(M, Nn, K, K, K, 0)
    assert want > 0, "a problem of this size takes the word-major scale copy when it can"
    outs = []
    for ws in (torch.empty(want, dtype=torch.uint8, device="cuda"), None):
        out = torch.empty((M, Nn), dtype=torch.bfloat16, device="cuda")
        N.check(lib.pt_gemm_mx(N.ptr(aq), N.ptr(as_), N.ptr(bq), N.ptr(bs), N.dtype_code(aq.dtype), 0, 0, N.ptr(out),
                               N.dtype_code(out.dtype), M, Nn, K, K, K, as_.shape[1], bs.shape[1], 0, N.ptr(ws),
                               0 if ws is None else ws.numel(), 0, N.stream_of(aq)))
        outs.append(out)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1])
    ref = OG.gemm_dequantized(Q.mx_dequant(codes_np(aq), codes_np(as_), "e4m3"), Q.mx_dequant(codes_np(bq), codes_np(bs), "e4m3"))
    _gate(ref, to_f32_np(outs[1]), "mxfp8 without workspace")


@pytest.mark.parametrize("tile_cfg", [0, 4])
def test_mx_gemm_exact_on_integers(tile_cfg):
    gi.TILE_CFG = tile_cfg
    try:
        _exact_on_integers((128, 128, 512) if tile_cfg == 0 else (384, 320, 1024))
    finally:
        gi.TILE_CFG = 0


def _exact_on_integers(shape):
    """Operands whose codes and block scales make every partial product an exact small integer
    times a power of two: the fp32 result must equal the exact value, which fails for any
    mismatch between scale bytes and the rows / K blocks they belong to."""
    M, N, K = shape
    rng = np.random.default_rng(64)
    # values k * 2^e with k in {-3..3} and a per (row, 32-block) exponent e in {-2..2}
    ea = rng.integers(-2, 3, size=(M, K // 32))
    eb = rng.integers(-2, 3, size=(N, K // 32))
    a = rng.integers(-3, 4, size=(M, K)) * np.exp2(np.repeat(ea, 32, axis=1))
    b = rng.integers(-3, 4, size=(N, K)) * np.exp2(np.repeat(eb, 32, axis=1))
    at, bt = torch.from_numpy(a).to(torch.bfloat16).cuda(), torch.from_numpy(b).to(torch.bfloat16).cuda()
    aq, as_ = qi.quantize_mxfp8_impl(at, torch.float8_e4m3fn, 1, 32)
    bq, bs = qi.quantize_mxfp8_impl(bt, torch.float8_e4m3fn, 1, 32)
    assert np.array_equal(Q.mx_dequant(codes_np(aq), codes_np(as_), "e4m3"), a.astype(np.float32))  # lossless
    out = gi.gemm_fp8_impl(aq, as_, False, bq, bs, True, torch.float32, False, G.MX_BLOCKWISE.value, 0)
    assert np.array_equal(to_f32_np(out).astype(np.float64), a @ b.T)
    if FP4 is not None:
        aq, as_ = qi.quantize_mxfp4_impl(at, FP4, 1, 32)
        bq, bs = qi.quantize_mxfp4_impl(bt, FP4, 1, 32)
        assert np.array_equal(Q.mx_dequant(codes_np(aq), codes_np(as_), "e2m1"), a.astype(np.float32))
        out = g4.gemm_fp4_impl(aq, as_, False, bq, bs, True, torch.float32, False, G.MX_BLOCKWISE.value, 0)
        assert np.array_equal(to_f32_np(out).astype(np.float64), a @ b.T)


@pytest.mark.parametrize("fmt", ["E4M3", "E5M2"])
def test_gemm_fp8_mx_autograd(fmt):
    M, N, K = 512, 768, 1024
    a = bf16_randn((M, K), seed=65).cuda().requires_grad_(True)
    b = bf16_randn((N, K), seed=66).cuda().requires_grad_(True)
    cfg = Float8QuantConfig(format=getattr(Format, fmt), granularity=G.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0)
    out = turbo.ops.gemm_fp8(a, b, trans_a=False, trans_b=True, out_dtype=torch.bfloat16, config=cfg)
    dy = bf16_randn((M, N), seed=67).cuda()
    out.backward(dy)
    torch.cuda.synchronize()
    af, bf_, dyf = to_f32_np(a), to_f32_np(b), to_f32_np(dy)
    gate = 25 if fmt == "E4M3" else 20
    assert OG.snr_db(af @ bf_.T, to_f32_np(out)) > gate
    assert OG.snr_db(dyf @ bf_, to_f32_np(a.grad)) > gate
    assert OG.snr_db(dyf.T @ af, to_f32_np(b.grad)) > gate


@pytest.mark.skipif(FP4 is None, reason="torch has no float4_e2m1fn_x2")
def test_gemm_fp4_autograd_and_main_grad():
    M, N, K = 512, 768, 1024
    a = bf16_randn((M, K), seed=68).cuda().requires_grad_(True)
    b = bf16_randn((N, K), seed=69).cuda().requires_grad_(True)
    out = turbo.ops.gemm_fp4(a, b, trans_a=False, trans_b=True, out_dtype=torch.bfloat16, config=Float4QuantConfig())
    dy = bf16_randn((M, N), seed=70).cuda()
    out.backward(dy)
    torch.cuda.synchronize()
    af, bf_, dyf = to_f32_np(a), to_f32_np(b), to_f32_np(dy)
    assert OG.snr_db(af @ bf_.T, to_f32_np(out)) > 10
    assert OG.snr_db(dyf @ bf_, to_f32_np(a.grad)) > 10
    assert OG.snr_db(dyf.T @ af, to_f32_np(b.grad)) > 10
    # fused accumulation of the weight gradient into an fp32 main_grad
    b2 = b.detach().clone().requires_grad_(True)
    b2.main_grad = torch.ones((N, K), dtype=torch.float32, device="cuda")
    b2.grad_added_to_main_grad = False
    a2 = a.detach().clone().requires_grad_(True)
    out2 = turbo.ops.gemm_fp4(a2, b2, trans_a=False, trans_b=True, out_dtype=torch.bfloat16, config=Float4QuantConfig(),
                              fuse_bgrad_accum_pattern="megatron")
    out2.backward(dy)
    torch.cuda.synchronize()
    assert b2.grad_added_to_main_grad
    got = (b2.main_grad - 1.0).cpu().numpy()
    assert OG.snr_db(to_f32_np(b.grad), got) > 40  # same product, bf16 vs fp32 output rounding
