"""GPU parity of the scaled FP8 GEMM.

Gate (from the path's accuracy target): against the fp32 matmul of the de-quantized
operands, max |err| / max |ref| <= 1e-2 and cosine >= 0.9999; plus the reference's SNR
gates against the unquantized matmul (25 dB E4M3, 20 dB E5M2) for the autograd wrappers.
"""

import numpy as np
import pytest
import torch

from helpers import FMT, bf16_randn, codes_np, gemm_gate, to_f32_np
from oracle import gemm as OG
from oracle import quantize as Q

pytestmark = pytest.mark.gpu

MAX_REL = 1e-2
MIN_COS = 0.9999


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, Float8QuantConfig, Format, ScalingRecipe, impl
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, Format, ScalingRecipe
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.kernels.gemm import gemm_fp8_impl as impl


def _gate(ref, got, what=""):
    return gemm_gate(ref, got, what)


def _deq_fp8(q: torch.Tensor, s: torch.Tensor, fmt):
    return Q.fp8_dequant(codes_np(q), to_f32_np(s), fmt)


# ----------------------------------------------------------------------------- impl level
@pytest.mark.parametrize("tile_cfg", [0, 1, 2, 3, 4])
@pytest.mark.parametrize(
    "M,N,K", [(256, 256, 128), (512, 384, 1024), (300, 200, 256), (1, 1, 128), (777, 130, 640), (4096, 4096, 512)]
)
def test_rowwise_and_tensorwise_nt(M, N, K, tile_cfg):
    if tile_cfg != 0 and M < 256:
        pytest.skip("pinned tile configs only on larger shapes")
    impl.TILE_CFG = tile_cfg
    try:
        a = bf16_randn((M, K), 31, scale=0.5)
        b = bf16_randn((N, K), 32, scale=0.5)
        for gran in (G.ROWWISE, G.TENSORWISE):
            kw = dict(axis=-1) if gran == G.ROWWISE else {}
            aq, asi = turbo.ops.quantize_fp8(a.cuda(), torch.float8_e4m3fn, gran, **kw)
            bq, bsi = turbo.ops.quantize_fp8(b.cuda(), torch.float8_e4m3fn, gran, **kw)
            c = impl.gemm_fp8_impl(aq, asi, False, bq, bsi, True, torch.bfloat16, False, gran.value, 0)
            torch.cuda.synchronize()
            ref = OG.gemm_dequantized(_deq_fp8(aq, asi, "e4m3"), _deq_fp8(bq, bsi, "e4m3"))
            assert c.shape == (M, N) and c.dtype == torch.bfloat16
            _gate(ref, to_f32_np(c), f"{gran.name} {M}x{N}x{K} cfg{tile_cfg}")
    finally:
        impl.TILE_CFG = 0


def test_exact_small_integers():
    """Integer-valued operands with unit scales: every product and partial sum is exact in
    fp32, so the kernel must reproduce the integer matmul bit for bit (catches any wrong
    operand byte order, swizzle or accumulator mapping)."""
    M, N, K = 384, 320, 512
    rng = np.random.default_rng(5)
    a = torch.from_numpy(rng.integers(-4, 5, (M, K)).astype(np.float32))
    b = torch.from_numpy(rng.integers(-4, 5, (N, K)).astype(np.float32))
    aq, bq = a.to(torch.float8_e4m3fn).cuda(), b.to(torch.float8_e4m3fn).cuda()
    one = torch.ones((), dtype=torch.float32, device="cuda")
    for cfg in (1, 2, 3):
        impl.TILE_CFG = cfg
        try:
            c = impl.gemm_fp8_impl(aq, one, False, bq, one, True, torch.float32, False, G.TENSORWISE.value, 0)
        finally:
            impl.TILE_CFG = 0
        assert torch.equal(c.cpu(), a @ b.t()), f"tile cfg {cfg}"
    # e5m2 and mixed formats (integers up to 4 are exact in e5m2 too)
    aq5, bq5 = a.to(torch.float8_e5m2).cuda(), b.to(torch.float8_e5m2).cuda()
    for x, y in ((aq5, bq5), (aq, bq5), (aq5, bq)):
        c = impl.gemm_fp8_impl(x, one, False, y, one, True, torch.float32, False, G.TENSORWISE.value, 0)
        assert torch.equal(c.cpu(), a @ b.t())


@pytest.mark.parametrize("trans_a,trans_b,trans_c", [(False, True, False), (False, False, False), (True, False, False),
                                                      (False, True, True), (True, False, True), (True, True, False)])
def test_layouts_rowwise(trans_a, trans_b, trans_c):
    M, N, K = 320, 448, 384
    a = bf16_randn((K, M) if trans_a else (M, K), 33)
    b = bf16_randn((N, K) if trans_b else (K, N), 34)
    aq, asi = turbo.ops.quantize_fp8(a.cuda(), torch.float8_e4m3fn, G.ROWWISE, axis=-2 if trans_a else -1)
    bq, bsi = turbo.ops.quantize_fp8(b.cuda(), torch.float8_e5m2, G.ROWWISE, axis=-1 if trans_b else -2)
    c = impl.gemm_fp8_impl(aq, asi, trans_a, bq, bsi, trans_b, torch.float16, trans_c, G.ROWWISE.value, 0)
    ref = OG.gemm_dequantized(_deq_fp8(aq, asi, "e4m3"), _deq_fp8(bq, bsi, "e5m2"), trans_a=trans_a, trans_b=trans_b)
    if trans_c:
        ref = ref.T
    assert tuple(c.shape) == ref.shape
    _gate(ref, to_f32_np(c), f"layout {trans_a}{trans_b}{trans_c}")


def test_blockwise_exact_small_integers():
    """Block-scaled kernels on integer operands with power-of-two block scales: every product,
    every scaled block sum and every partial sum is exact in fp32, so each tile configuration
    has to give the integer result bit for bit (wrong row / block of a scale, a wrong fragment
    or accumulator mapping, a slab applied twice or dropped at a tile change all show)."""
    M, N, K = 768, 640, 1024
    rng = np.random.default_rng(6)
    a = torch.from_numpy(rng.integers(-4, 5, (M, K)).astype(np.float32))
    b = torch.from_numpy(rng.integers(-4, 5, (N, K)).astype(np.float32))
    sa = torch.from_numpy(np.exp2(rng.integers(-3, 4, (M, K // 128))).astype(np.float32))
    sb = torch.from_numpy(np.exp2(rng.integers(-3, 4, ((N + 127) // 128, K // 128))).astype(np.float32))
    ad = a * sa.repeat_interleave(128, dim=1)
    bd = b * sb.repeat_interleave(128, dim=0)[:N].repeat_interleave(128, dim=1)
    want = ad.double() @ bd.double().t()
    assert want.abs().max() < 2**24
    aq, bq = a.to(torch.float8_e4m3fn).cuda(), b.to(torch.float8_e4m3fn).cuda()
    for cfg in (1, 2, 3, 4):
        impl.TILE_CFG = cfg
        try:
            c = impl.gemm_fp8_impl(aq, sa.cuda(), False, bq, sb.cuda(), True, torch.float32, False, G.BLOCKWISE.value, 0)
        finally:
            impl.TILE_CFG = 0
        assert torch.equal(c.cpu().double(), want), f"tile cfg {cfg}"


@pytest.mark.parametrize("tile_cfg", [0, 4])
@pytest.mark.parametrize("M,N,K", [(512, 384, 512), (300, 260, 256), (2048, 1024, 1024), (16384, 1024, 256)])
def test_blockwise_nt_nn_tn(M, N, K, tile_cfg):
    impl.TILE_CFG = tile_cfg
    try:
        _blockwise_nt_nn_tn(M, N, K)
    finally:
        impl.TILE_CFG = 0


def _blockwise_nt_nn_tn(M, N, K):
    a = bf16_randn((M, K), 35, outlier_frac=0.001)
    w = bf16_randn((N, K), 36)
    f8 = torch.float8_e4m3fn
    a_row, a_rs, a_col, a_cs = turbo.ops.quantize_fp8_with_trans(a.cuda(), f8, G.BLOCKWISE, block_size=128)
    wq, ws = turbo.ops.quantize_fp8(w.cuda(), f8, G.BLOCKWISE, block_size=128, scaling_recipe=ScalingRecipe(True))
    a_row_d = Q.fp8_blockwise_dequant(codes_np(a_row), to_f32_np(a_rs), 1)
    a_col_d = Q.fp8_blockwise_dequant(codes_np(a_col), to_f32_np(a_cs), 0)
    w_d = Q.fp8_blockwise_weight_dequant(codes_np(wq), to_f32_np(ws))
    # NT forward: [M,K] x [N,K]^T
    c = impl.gemm_fp8_impl(a_row, a_rs, False, wq, ws, True, torch.bfloat16, False, G.BLOCKWISE.value, 0)
    _gate(OG.gemm_dequantized(a_row_d, w_d), to_f32_np(c), "blockwise NT")
    # NN dgrad: grad [M,N] x W [N,K] -> [M,K]
    g = bf16_randn((M, N), 37)
    g_row, g_rs, g_col, g_cs = turbo.ops.quantize_fp8_with_trans(g.cuda(), f8, G.BLOCKWISE, block_size=128)
    g_row_d = Q.fp8_blockwise_dequant(codes_np(g_row), to_f32_np(g_rs), 1)
    g_col_d = Q.fp8_blockwise_dequant(codes_np(g_col), to_f32_np(g_cs), 0)
    da = impl.gemm_fp8_impl(g_row, g_rs, False, wq, ws, False, torch.bfloat16, False, G.BLOCKWISE.value, 0)
    _gate(OG.gemm_dequantized(g_row_d, w_d, trans_b=False), to_f32_np(da), "blockwise NN")
    # TN wgrad: A_col^T [K,M] x grad_col [M,N] -> [K,N]; trans_c gives dW [N,K]
    dw = impl.gemm_fp8_impl(a_col, a_cs, True, g_col, g_cs, False, torch.bfloat16, True, G.BLOCKWISE.value, 0)
    ref = OG.gemm_dequantized(a_col_d, g_col_d, trans_a=True, trans_b=False).T
    assert tuple(dw.shape) == (N, K)
    _gate(ref, to_f32_np(dw), "blockwise TN^T")


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M", [256, 200])
def test_accumulate_epilogue(out_dtype, M):
    """out += A B^T for every output type (16-bit outputs add in fp32 and round once); M = 200 leaves
    row groups of the last tile outside the matrix."""
    N, K = 384, 256
    a, b = bf16_randn((M, K), 38), bf16_randn((N, K), 39)
    aq, asi = turbo.ops.quantize_fp8(a.cuda(), torch.float8_e4m3fn, G.TENSORWISE)
    bq, bsi = turbo.ops.quantize_fp8(b.cuda(), torch.float8_e4m3fn, G.TENSORWISE)
    base = (bf16_randn((M, N), 40).float() * 8).to(out_dtype)
    out = base.cuda().clone()
    impl.gemm_fp8_accum_impl(aq, asi, False, bq, bsi, True, out_dtype, False, G.TENSORWISE.value, out, 0)
    prod = OG.gemm_dequantized(_deq_fp8(aq, asi, "e4m3"), _deq_fp8(bq, bsi, "e4m3"))
    ref = prod + base.float().numpy()
    _gate(ref, out.float().cpu().numpy(), f"accumulate {out_dtype}")
    # the old values really took part: without them the result is off by their norm
    plain = torch.empty_like(out)
    impl.gemm_fp8_accum_impl(aq, asi, False, bq, bsi, True, out_dtype, False, G.TENSORWISE.value, plain.zero_(), 0)
    diff = (out.float() - plain.float()).cpu().numpy()
    assert np.abs(diff - base.float().numpy()).max() <= 2.0 ** -6 * max(1.0, float(np.abs(ref).max()))


def test_determinism():
    a, b = bf16_randn((1024, 1024), 41), bf16_randn((768, 1024), 42)
    cfg = Float8QuantConfig(granularity=G.BLOCKWISE, block_size=128)
    outs = [turbo.ops.gemm_fp8(a.cuda(), b.cuda(), trans_b=True, out_dtype=torch.bfloat16, config=cfg) for _ in range(10)]
    for o in outs[1:]:
        assert torch.equal(o, outs[0])


# ----------------------------------------------------------------------------- autograd level
def _snr_ok(ref, got, fmt):
    snr = OG.snr_db(to_f32_np(ref), to_f32_np(got))
    assert snr > (25 if fmt == Format.E4M3 else 20), f"SNR {snr:.1f} dB"


@pytest.mark.parametrize("fmt", ["E4M3", "E5M2", "HYBRID"])
@pytest.mark.parametrize("gran", ["TENSORWISE", "ROWWISE", "BLOCKWISE"])
@pytest.mark.parametrize("trans_b", [True, False])
def test_gemm_fp8_autograd(gran, fmt, trans_b):
    fmt_e, gran_e = Format[fmt], G[gran]
    M, N, K = 512, 384, 640
    cfg = Float8QuantConfig(format=fmt_e, granularity=gran_e, block_size=128 if gran_e == G.BLOCKWISE else None)
    a = bf16_randn((M, K), 43).cuda().requires_grad_(True)
    b = bf16_randn((N, K) if trans_b else (K, N), 44).cuda().requires_grad_(True)
    out = turbo.ops.gemm_fp8(a, b, trans_a=False, trans_b=trans_b, out_dtype=torch.bfloat16, config=cfg)
    go = bf16_randn((M, N), 45).cuda()
    out.backward(go)
    a_ref = a.detach().clone().requires_grad_(True)
    b_ref = b.detach().clone().requires_grad_(True)
    out_ref = a_ref @ (b_ref.t() if trans_b else b_ref)
    out_ref.backward(go)
    gate_fmt = Format.E5M2 if fmt_e == Format.E5M2 else Format.E4M3
    _snr_ok(out_ref, out, gate_fmt)
    _snr_ok(a_ref.grad, a.grad, Format.E5M2 if fmt_e != Format.E4M3 else Format.E4M3)
    _snr_ok(b_ref.grad, b.grad, Format.E5M2 if fmt_e != Format.E4M3 else Format.E4M3)
    assert a.grad.shape == a.shape and b.grad.shape == b.shape


def test_prequantized_operands_and_fused_main_grad():
    from primus_turbo.pytorch.core.quantized_tensor import QuantizedTensor

    M, N, K = 256, 256, 384
    a = bf16_randn((M, K), 46).cuda()
    b = bf16_randn((N, K), 47).cuda()
    cfg = Float8QuantConfig(granularity=G.ROWWISE)
    qa = QuantizedTensor.quantize(a, torch.float8_e4m3fn, G.ROWWISE, axis=-1)
    qb = QuantizedTensor.quantize(b, torch.float8_e4m3fn, G.ROWWISE, axis=-1)
    out_q = turbo.ops.gemm_fp8(qa, qb, trans_b=True, out_dtype=torch.bfloat16, config=cfg)
    out = turbo.ops.gemm_fp8(a, b, trans_b=True, out_dtype=torch.bfloat16, config=cfg)
    assert torch.equal(out_q, out)
    # fused wgrad accumulation (TENSORWISE): main_grad receives += dW, returned grad is a dummy
    w = torch.nn.Parameter(b.clone())
    w.main_grad = torch.zeros_like(w, dtype=torch.float32)
    w.grad_added_to_main_grad = False
    x = a.clone().requires_grad_(True)
    y = turbo.ops.gemm_fp8(x, w, trans_b=True, out_dtype=torch.bfloat16, fuse_bgrad_accum_pattern="megatron")
    go = bf16_randn((M, N), 48).cuda()
    y.backward(go)
    assert w.grad_added_to_main_grad is True
    ref_dw = go.float().t() @ a.float()
    assert OG.snr_db(ref_dw.cpu().numpy(), w.main_grad.cpu().numpy()) > 25
    y2 = turbo.ops.gemm_fp8(x, w, trans_b=True, out_dtype=torch.bfloat16, fuse_bgrad_accum_pattern="megatron")
    y2.backward(go)
    assert OG.snr_db(2 * ref_dw.cpu().numpy(), w.main_grad.cpu().numpy()) > 25
