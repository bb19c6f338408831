"""GPU parity: FP8 128-blockwise quantizers vs the CPU oracle (bit-exact bytes and scales)."""

import numpy as np
import pytest
import torch

from helpers import FMT, bf16_randn, bits_np, codes_np, round_to, to_f32_np, group_lens
from oracle import quantize as Q

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, ScalingRecipe
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.core.low_precision import ScalingRecipe


def _eq_scales(got: torch.Tensor, want: np.ndarray):
    assert tuple(got.shape) == want.shape, (got.shape, want.shape)
    assert np.array_equal(bits_np(got), want.view(np.uint32))


SHAPES = [(16384, 2048), (256, 256), (128, 128), (1, 1), (1, 300), (300, 1), (129, 257), (200, 128), (555, 1000), (64, 4104)]


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("shape", SHAPES)
def test_blockwise_row_col_dual(shape, dtype):
    if shape[0] == 16384 and dtype != torch.float8_e4m3fn:
        pytest.skip("headline size only for e4m3")
    x = bf16_randn(shape, seed=21, outlier_frac=0.001)
    xf = to_f32_np(x)
    xg = x.cuda()
    f = FMT[dtype]
    oqr, osr = Q.fp8_blockwise(xf, 1, f)
    oqc, osc = Q.fp8_blockwise(xf, 0, f)
    q, s = turbo.ops.quantize_fp8(xg, dtype, G.BLOCKWISE, block_size=128, axis=1)
    assert np.array_equal(codes_np(q), oqr)
    _eq_scales(s, osr)
    q0, s0 = turbo.ops.quantize_fp8(xg, dtype, G.BLOCKWISE, block_size=128, axis=0)
    assert np.array_equal(codes_np(q0), oqc)
    _eq_scales(s0, osc)
    qr, sr, qc, sc = turbo.ops.quantize_fp8_with_trans(xg, dtype, G.BLOCKWISE, block_size=128)
    assert np.array_equal(codes_np(qr), oqr) and np.array_equal(codes_np(qc), oqc)
    _eq_scales(sr, osr)
    _eq_scales(sc, osc)
    # negative axis aliases
    qn, sn = turbo.ops.quantize_fp8(xg, dtype, G.BLOCKWISE, block_size=128, axis=-2)
    assert torch.equal(qn.view(torch.uint8), q0.view(torch.uint8)) and torch.equal(sn, s0)
    # de-quantize both directions
    y1 = turbo.ops.dequantize_fp8(q, torch.bfloat16, G.BLOCKWISE, block_size=128, axis=1, scale_inv=s)
    assert np.array_equal(bits_np(y1), bits_np(round_to(Q.fp8_blockwise_dequant(oqr, osr, 1, f), torch.bfloat16)))
    y0 = turbo.ops.dequantize_fp8(q0, torch.float32, G.BLOCKWISE, block_size=128, axis=0, scale_inv=s0)
    assert np.array_equal(bits_np(y0), Q.fp8_blockwise_dequant(oqc, osc, 0, f).view(np.uint32))
    # every full-magnitude block holds a code of magnitude qmax (0x7E e4m3 / 0x7B e5m2)
    top = 0x7E if dtype == torch.float8_e4m3fn else 0x7B
    if shape[1] % 128 == 0:
        blocks = (codes_np(q) & 0x7F).reshape(shape[0], -1, 128).max(axis=2)
        amax = np.abs(xf).reshape(shape[0], -1, 128).max(axis=2)
        assert np.all(blocks[amax >= 1e-4] == top)


def test_blockwise_rows_alone_random_shapes():
    """Forty random shapes (columns a multiple of 8): the row blocks quantized alone (streaming
    kernel), in both scale layouts, give the bytes and scales of the dual quantizer's row output."""
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

    rng = np.random.default_rng(61)
    for k in range(40):
        M, N = int(rng.integers(1, 701)), 8 * int(rng.integers(1, 601))
        src = (torch.bfloat16, torch.float16, torch.float32)[k % 3]
        x = bf16_randn((M, N), seed=700 + k, outlier_frac=0.001, dtype=src).cuda()
        dt = torch.float8_e5m2 if k % 4 == 3 else torch.float8_e4m3fn
        qr, sr, _, _ = turbo.ops.quantize_fp8_with_trans(x, dt, G.BLOCKWISE, block_size=128)
        q, s = turbo.ops.quantize_fp8(x, dt, G.BLOCKWISE, block_size=128, axis=1)
        assert torch.equal(q.view(torch.uint8), qr.view(torch.uint8)) and torch.equal(s, sr), (M, N, src)
        q2, s_km, _, _ = qi.quant_fp8_blockwise_kmajor_impl(x, dt, 128, False)
        assert torch.equal(q2.view(torch.uint8), qr.view(torch.uint8)) and torch.equal(s_km.t().contiguous(), sr), (M, N, src)


@pytest.mark.parametrize("src", [torch.float16, torch.float32])
def test_blockwise_other_sources(src):
    x = bf16_randn((300, 520), 22, dtype=src)
    qr, sr, qc, sc = turbo.ops.quantize_fp8_with_trans(x.cuda(), torch.float8_e4m3fn, G.BLOCKWISE, block_size=128)
    oqr, osr, oqc, osc = Q.fp8_blockwise_dual(to_f32_np(x), "e4m3")
    assert np.array_equal(codes_np(qr), oqr) and np.array_equal(codes_np(qc), oqc)
    _eq_scales(sr, osr)
    _eq_scales(sc, osc)
    q, s = turbo.ops.quantize_fp8(x.cuda(), torch.float8_e4m3fn, G.BLOCKWISE, block_size=128, axis=1)  # rows alone
    assert np.array_equal(codes_np(q), oqr)
    _eq_scales(s, osr)


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("shape", [(7168, 2048), (4, 512, 384), (2, 130, 260), (100, 100), (3, 1, 1), (32, 4096, 7168)])
def test_blockwise_weight(shape, dtype):
    if shape[0] in (32, 7168) and dtype != torch.float8_e4m3fn:
        pytest.skip("large size only for e4m3")
    x = bf16_randn(shape, seed=23)
    f = FMT[dtype]
    rec = ScalingRecipe(use_2d_block=True)
    q, s = turbo.ops.quantize_fp8(x.cuda(), dtype, G.BLOCKWISE, block_size=128, scaling_recipe=rec)
    torch.cuda.synchronize()
    oq, os_ = Q.fp8_blockwise_weight(to_f32_np(x), f)
    assert np.array_equal(codes_np(q), oq)
    _eq_scales(s, os_)
    if shape[0] != 32:
        y = turbo.ops.dequantize_fp8(q, torch.bfloat16, G.BLOCKWISE, block_size=128, scale_inv=s, scaling_recipe=rec)
        want = round_to(Q.fp8_blockwise_weight_dequant(oq, os_, f), torch.bfloat16)
        assert np.array_equal(bits_np(y), bits_np(want))


@pytest.mark.parametrize(
    "kind,G_,M,N",
    [
        ("balanced", 4, 1024, 512),
        ("ragged", 8, 3000, 384),
        ("zeros", 8, 16384, 256),
        ("zipf", 32, 32768, 2048),
        ("ragged", 3, 77, 100),
        ("zipf", 32, 8192, 7168),
    ],
)
def test_grouped_segment_row_col(kind, G_, M, N):
    lens = group_lens(kind, G_, M, 24)
    assert lens.sum() == M
    x = bf16_randn((M, N), seed=25, outlier_frac=0.001)
    gl = torch.from_numpy(lens).cuda()
    offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)
    assert np.array_equal(offs.cpu().numpy(), Q.group_offs(lens))
    from primus_turbo.pytorch.kernels.quantization.quantization_impl import (
        quant_fp8_blockwise_segment_m_row_col_impl as seg,
    )

    qr, qc, sr, sc, plens, poffs = seg(x.cuda(), torch.float8_e4m3fn, 128, gl, offs, N)
    torch.cuda.synchronize()
    o = Q.fp8_blockwise_segment_m_row_col(to_f32_np(x), lens, "e4m3")
    assert np.array_equal(plens.cpu().numpy(), o["padded_lens"])
    assert np.array_equal(poffs.cpu().numpy(), o["padded_offs"])
    assert np.array_equal(codes_np(qr), o["row"])
    _eq_scales(sr, o["row_scale"])
    w = o["written_rows"]
    assert tuple(qc.shape) == o["col"].shape and tuple(sc.shape) == o["col_scale"].shape
    assert np.array_equal(codes_np(qc)[:w], o["col"][:w])
    assert np.array_equal(bits_np(sc)[: w // 128], o["col_scale"].view(np.uint32)[: w // 128])
    # row scales are the plain 1x128 scales transposed
    _, s_plain = turbo.ops.quantize_fp8(x.cuda(), torch.float8_e4m3fn, G.BLOCKWISE, block_size=128, axis=1)
    assert torch.equal(sr, s_plain.t().contiguous())


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("shape", [(7168, 2048), (4, 512, 384), (2, 144, 260), (112, 100), (3, 16, 8), (8, 4096, 1024)])
def test_blockwise_weight_dual_transposed_copy(shape, dtype):
    """The dual weight quantizer: codes and scales identical to the plain one, and the second output
    is exactly the transpose of the codes (per batch slice)."""
    from primus_turbo.pytorch.kernels.quantization.quantization_impl import quant_fp8_blockwise_for_weight_dual_impl as dual

    x = bf16_randn(shape, seed=26).cuda()
    q, s = turbo.ops.quantize_fp8(x, dtype, G.BLOCKWISE, block_size=128, scaling_recipe=ScalingRecipe(use_2d_block=True))
    q2, qt, s2 = dual(x, dtype, 128)
    torch.cuda.synchronize()
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2, s)
    assert qt.shape == x.shape[:-2] + (x.shape[-1], x.shape[-2])
    assert torch.equal(qt.view(torch.uint8), q.view(torch.uint8).transpose(-2, -1).contiguous())
    with pytest.raises(RuntimeError, match="multiple of 16"):
        dual(bf16_randn((100, 128), seed=1).cuda(), dtype, 128)


@pytest.mark.parametrize("kind,G_,M,N", [("balanced", 4, 1024, 512), ("ragged", 8, 3000, 384), ("zeros", 8, 16384, 256),
                                         ("ragged", 3, 77, 104), ("zipf", 32, 8192, 7168)])
@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_grouped_segment_row_col_transposed(kind, G_, M, N, dtype):
    """The grouped quantizer with the column codes emitted transposed: everything equals the plain
    variant, the transposed codes are its column output transposed (up to the last padded group)."""
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

    lens = group_lens(kind, G_, M, 27)
    x = bf16_randn((M, N), seed=28, outlier_frac=0.001).cuda()
    gl = torch.from_numpy(lens).cuda()
    offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)
    qr, qc, sr, sc, plens, poffs = qi.quant_fp8_blockwise_segment_m_row_col_impl(x, dtype, 128, gl, offs, N)
    qr2, qct, sr2, sc2, plens2, poffs2 = qi.quant_fp8_blockwise_segment_m_row_col_t_impl(x, dtype, 128, gl, offs)
    torch.cuda.synchronize()
    w = int(poffs[-1])
    assert torch.equal(qr2.view(torch.uint8), qr.view(torch.uint8)) and torch.equal(sr2, sr)
    assert torch.equal(plens2, plens) and torch.equal(poffs2, poffs)
    assert torch.equal(sc2[: w // 128], sc[: w // 128])
    assert qct.shape == (N, -(-(M + 128 * G_) // 128) * 128)
    assert torch.equal(qct.view(torch.uint8)[:, :w], qc.view(torch.uint8)[:w].t().contiguous())


@pytest.mark.parametrize("shape", [(256, 384), (130, 257), (1000, 512), (16384, 2048), (77, 96)])
@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_blockwise_dual_transposed_column_output(shape, dtype):
    """Dual quantizer with the column codes emitted transposed: rows / scales identical to the plain
    dual quantizer, transposed codes = its column codes transposed, zero beyond M."""
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

    M, N = shape
    x = bf16_randn(shape, seed=29, outlier_frac=0.001).cuda()
    qr, sr, qc, sc = qi.quant_fp8_blockwise_dual_impl(x, dtype, 128)
    qr2, sr2, qct, sc2 = qi.quant_fp8_blockwise_dual_t_impl(x, dtype, 128)
    torch.cuda.synchronize()
    Mp = -(-M // 128) * 128
    assert torch.equal(qr2.view(torch.uint8), qr.view(torch.uint8)) and torch.equal(sr2, sr) and torch.equal(sc2, sc)
    assert qct.shape == (N, Mp)
    assert torch.equal(qct.view(torch.uint8)[:, :M], qc.view(torch.uint8).t().contiguous())
    assert not bool(qct.view(torch.uint8)[:, M:].any())


@pytest.mark.parametrize("shape", [(256, 384), (130, 257), (1000, 512), (16384, 2048), (77, 96), (1, 1)])
@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("with_col_t", [False, True])
def test_blockwise_row_scales_block_major(shape, dtype, with_col_t):
    """The quantizer that stores its row scales block-major ([N/128, M], the layout the block-scaled
    GEMM reads): codes and scale values bit for bit those of the oracle, the optional transposed
    column output that of the dual quantizer; and the GEMM gives identical bits whether it gets the
    [M, N/128] view of these scales or a contiguous copy of it."""
    from primus_turbo.pytorch.kernels.gemm import gemm_fp8_impl as gi
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

    M, N = shape
    x = bf16_randn(shape, seed=27, outlier_frac=0.001)
    xf, f = to_f32_np(x), FMT[dtype]
    q, s_km, q_t, s_col = qi.quant_fp8_blockwise_kmajor_impl(x.cuda(), dtype, 128, with_col_t)
    torch.cuda.synchronize()
    oq, os_ = Q.fp8_blockwise(xf, 1, f)
    assert np.array_equal(codes_np(q), oq)
    assert s_km.is_contiguous() and tuple(s_km.shape) == (os_.shape[1], M)
    _eq_scales(s_km.t().contiguous(), os_)
    if with_col_t:
        oqc, osc = Q.fp8_blockwise(xf, 0, f)
        assert np.array_equal(codes_np(q_t)[:, :M], oqc.T) and not codes_np(q_t)[:, M:].any()
        _eq_scales(s_col, osc)
    else:
        assert q_t.numel() == 0 and s_col.numel() == 0
    if N >= 256 and M >= 77:
        w = bf16_randn((192, N), seed=28).cuda()
        wq, ws = qi.quant_fp8_blockwise_for_weight_impl(w, torch.float8_e4m3fn, 128)
        a = gi.gemm_fp8_impl(q, s_km.t(), False, wq, ws, True, torch.bfloat16, False, G.BLOCKWISE.value, 0)
        b = gi.gemm_fp8_impl(q, s_km.t().contiguous(), False, wq, ws, True, torch.bfloat16, False, G.BLOCKWISE.value, 0)
        c = gi.gemm_fp8_impl(q, s_km.t(), False, wq, ws, True, torch.bfloat16, True, G.BLOCKWISE.value, 0)
        torch.cuda.synchronize()
        assert torch.equal(a, b) and torch.equal(c, a.t().contiguous())
