"""GPU parity of the grouped MXFP4 path (MoE experts, E2M1 codes with E8M0 block scales): the grouped
quantizer (rows in place, transposed column direction padded to 256 tokens per group) bit for bit
against the oracle; the row-group GEMM and the variable-K wgrad GEMM against the fp32 matmul of the
de-quantized operands (max |err| / max |ref| <= 1e-2, cosine >= 0.9999), including N / K that are
multiples of 32 only; the autograd op at the reference's SNR gate of 8 dB
(tests/pytorch/ops/test_grouped_gemm_fp4.py:54-56 of the reference), its empty-expert and
fused-accumulation cases (same file: 246-330, 341-400)."""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, codes_np, gemm_gate, group_lens, to_f32_np
from oracle import gemm as OG
from oracle import quantize as Q

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, Float4QuantConfig, ScalingRecipe, gimpl, qimpl, FP4
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig, ScalingRecipe, float4_e2m1fn_x2 as FP4
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.kernels.grouped_gemm import grouped_gemm_fp4_impl as gimpl
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qimpl


def _gate(ref, got, what=""):
    return gemm_gate(ref, got, what)


def _offs(lens):
    gl = torch.from_numpy(np.asarray(lens, dtype=np.int64)).cuda()
    return gl, torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)


def _oracle(x, lens):
    return Q.mx_grouped_quant(x.float().numpy(), lens, "e2m1", row_align=1, col_align=256)


QCASES = [("balanced", 4, 512, 256), ("ragged", 8, 1000, 384), ("zeros", 8, 640, 128), ("zipf", 32, 4096, 512),
          ("ragged", 3, 77, 96), ("balanced", 1, 200, 160)]


@pytest.mark.parametrize("kind,G_,M,N", QCASES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_grouped_mxfp4_quantizer_bit_exact(kind, G_, M, N, dtype):
    lens = group_lens(kind, G_, M, 61)
    gl, offs = _offs(lens)
    x = bf16_randn((M, N), seed=62, outlier_frac=0.002).to(dtype)
    rq, rs, cq, cs, lr, orow, lc, ocol = qimpl.grouped_quantize_mxfp4_impl(x.cuda(), FP4, None, 32, gl, offs, with_trans=True)
    o = _oracle(x, lens)
    n_pad, mc_alloc = -(-N // 128) * 128, -(-(M + 256 * G_) // 256) * 256
    assert rq.shape == (M, n_pad // 2) and rs.shape == (M, n_pad // 32)
    assert cq.shape == (N, mc_alloc // 2) and cs.shape == (N, mc_alloc // 32)
    assert torch.equal(lr, gl) and torch.equal(orow, offs)  # rows stay in place
    assert np.array_equal(lc.cpu().numpy(), o["col_lens"]) and np.array_equal(ocol.cpu().numpy(), o["col_offs"])
    mc = int(o["col_offs"][-1])
    assert np.array_equal(codes_np(rq), o["row"]) and np.array_equal(codes_np(rs), o["row_scale"])
    assert np.array_equal(codes_np(cq)[:, : mc // 2], o["col"]) and np.array_equal(codes_np(cs)[:, : mc // 32], o["col_scale"])
    # the row direction is the dense row quantizer
    dq, dsc = qimpl.quantize_mxfp4_impl(x.cuda(), FP4, 1, 32)
    assert torch.equal(dq.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(dsc.view(torch.uint8), rs.view(torch.uint8))
    # one direction at a time gives the same tensors
    q1, s1, l1, o1 = qimpl.grouped_quantize_mxfp4_impl(x.cuda(), FP4, 1, 32, gl, offs)
    q0, s0, l0, o0 = qimpl.grouped_quantize_mxfp4_impl(x.cuda(), FP4, 0, 32, gl, offs)
    assert np.array_equal(codes_np(q1), o["row"]) and np.array_equal(codes_np(s1), o["row_scale"])
    assert np.array_equal(codes_np(q0)[:, : mc // 2], o["col"]) and np.array_equal(codes_np(s0)[:, : mc // 32], o["col_scale"])
    assert torch.equal(o1, offs) and torch.equal(o0, ocol) and torch.equal(l1, gl) and torch.equal(l0, lc)


@pytest.mark.parametrize("kind,G_,M,N", [("ragged", 8, 1000, 384), ("zeros", 8, 640, 128), ("ragged", 3, 77, 96)])
def test_grouped_mxfp4_quantizer_2d_blocks_bit_exact(kind, G_, M, N):
    """32 x 32 blocks in the grouped MXFP4 quantizer, counted from each group's first row (row
    direction: rows stay where they are; column direction: groups padded to 256)."""
    lens = group_lens(kind, G_, M, 63)
    gl, offs = _offs(lens)
    x = bf16_randn((M, N), seed=64, outlier_frac=0.002)
    rec = ScalingRecipe(use_2d_block=True)
    rq, rs, cq, cs, _, _, _, ocol = qimpl.grouped_quantize_mxfp4_impl(x.cuda(), FP4, None, 32, gl, offs, with_trans=True,
                                                                      scaling_recipe=rec, scaling_recipe_for_trans=rec)
    o = Q.mx_grouped_quant(to_f32_np(x), lens, "e2m1", row_align=1, col_align=256, row_2d=True, col_2d=True)
    mc = int(o["col_offs"][-1])
    assert np.array_equal(ocol.cpu().numpy(), o["col_offs"])
    assert np.array_equal(codes_np(rs), o["row_scale"]) and np.array_equal(codes_np(rq), o["row"])
    assert np.array_equal(codes_np(cs)[:, : mc // 32], o["col_scale"]) and np.array_equal(codes_np(cq)[:, : mc // 2], o["col"])


# (kind, G, M, N, K): includes N / K that are multiples of 32 only and K below four slabs
GCASES = [("balanced", 4, 1024, 512, 1024), ("ragged", 8, 3000, 384, 2048), ("zeros", 8, 2048, 256, 1024),
          ("zipf", 32, 8192, 1024, 1536), ("ragged", 3, 77, 96, 160), ("zipf", 16, 4096, 2048, 1408),
          ("ragged", 4, 500, 288, 256), ("balanced", 2, 256, 1568, 2080)]


@pytest.mark.parametrize("kind,G_,M,N,K", GCASES)
def test_grouped_mxfp4_forward_product(kind, G_, M, N, K):
    lens = group_lens(kind, G_, M, 63)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=64)
    w = bf16_randn((G_, N, K), seed=65)
    rq, rs, _, orow = qimpl.grouped_quantize_mxfp4_impl(x.cuda(), FP4, 1, 32, gl, offs)
    wq, ws = qimpl.quantize_mxfp4_impl(w.cuda(), FP4, 2, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))
    out = gimpl.grouped_gemm_fp4_impl(rq, wq, rs, ws, gl, orow, False, True, torch.bfloat16, G.MX_BLOCKWISE.value, None, 0,
                                      False, offs)
    torch.cuda.synchronize()
    assert out.shape == (M, N)
    a_deq = Q.mx_dequant(codes_np(rq), codes_np(rs), "e2m1")[:, :K]
    w_deq = np.stack([Q.mx_dequant(codes_np(wq[g]), codes_np(ws[g]), "e2m1")[:, :K] for g in range(G_)])
    ref = OG.grouped_gemm_dequantized(a_deq, w_deq, lens, trans_b=True)
    _gate(ref, to_f32_np(out), f"{kind} G={G_} {M}x{N}x{K}")


@pytest.mark.parametrize("kind,G_,M,N,K", [("zipf", 32, 8192, 1024, 768), ("ragged", 8, 3000, 384, 1024), ("zeros", 8, 2048, 256, 512),
                                           ("ragged", 3, 77, 96, 640), ("zipf", 16, 4096, 2048, 2048)])
def test_grouped_mxfp4_eight_wavefront_tile(kind, G_, M, N, K):
    """tile_cfg 4 (256 x 256 tile, eight wavefronts, row groups) against the automatic configuration:
    the same products in the same order, so the same bits."""
    from primus_turbo.pytorch.kernels.grouped_gemm import grouped_gemm_fp8_impl as g8

    lens = group_lens(kind, G_, M, 163)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=164).cuda()
    w = bf16_randn((G_, N, K), seed=165).cuda()
    rq, rs, _, orow = qimpl.grouped_quantize_mxfp4_impl(x, FP4, 1, 32, gl, offs)
    wq, ws = qimpl.quantize_mxfp4_impl(w, FP4, 2, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))
    run = lambda: gimpl.grouped_gemm_fp4_impl(rq, wq, rs, ws, gl, orow, False, True, torch.bfloat16, G.MX_BLOCKWISE.value,  # noqa: E731
                                              None, 0, False, offs)
    auto = run()
    g8.MX_TILE_CFG = 4
    try:
        got = run()
    finally:
        g8.MX_TILE_CFG = 0
    torch.cuda.synchronize()
    assert torch.equal(got, auto)


@pytest.mark.parametrize("kind,G_,M,N,K", GCASES)
@pytest.mark.parametrize("trans_c", [False, True])
def test_grouped_mxfp4_variable_k_product(kind, G_, M, N, K, trans_c):
    lens = group_lens(kind, G_, M, 66)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=67)
    dy = bf16_randn((M, N), seed=68)
    xq, xs, lc, ocol = qimpl.grouped_quantize_mxfp4_impl(x.cuda(), FP4, 0, 32, gl, offs)
    gq, gs, _, _ = qimpl.grouped_quantize_mxfp4_impl(dy.cuda(), FP4, 0, 32, gl, offs)
    out = gimpl.grouped_gemm_fp4_variable_k_impl(gq, xq, gs, xs, lc, ocol, False, False, trans_c, torch.float32,
                                                 G.MX_BLOCKWISE.value, None, 0)
    torch.cuda.synchronize()
    assert out.shape == ((G_, K, N) if trans_c else (G_, N, K))
    ox, og = _oracle(x, lens), _oracle(dy, lens)
    xd = Q.mx_dequant(ox["col"], ox["col_scale"], "e2m1")  # [K, Mc]
    gd = Q.mx_dequant(og["col"], og["col_scale"], "e2m1")  # [N, Mc]
    co = ox["col_offs"]
    ref = np.stack([gd[:, co[g] : co[g + 1]].astype(np.float64) @ xd[:, co[g] : co[g + 1]].astype(np.float64).T
                    for g in range(G_)]).astype(np.float32)
    if trans_c:
        ref = np.ascontiguousarray(ref.transpose(0, 2, 1))
    _gate(ref, to_f32_np(out), f"variable-K {kind} G={G_}")
    for g in range(G_):
        if lens[g] == 0:
            assert not bool(out[g].abs().max() > 0)
    # beta = 1 epilogue
    acc = torch.ones_like(out)
    gimpl.grouped_gemm_fp4_variable_k_accum_impl(gq, xq, gs, xs, lc, ocol, False, False, trans_c, torch.float32,
                                                 G.MX_BLOCKWISE.value, None, 0, acc)
    assert torch.allclose(acc, out + 1, rtol=0, atol=1e-3 * float(out.abs().max()) + 1e-6)


def _autograd_case(lens, N, K, dtype, seed):
    G_, M = len(lens), int(np.sum(lens))
    gl, _ = _offs(lens)
    a = bf16_randn((M, K), seed=seed).to(dtype).cuda().requires_grad_(True)
    b = bf16_randn((G_, N, K), seed=seed + 1).to(dtype).cuda().requires_grad_(True)
    out = turbo.ops.grouped_gemm_fp4(a, b, gl, trans_b=True, config=Float4QuantConfig())
    assert out.shape == (M, N) and out.dtype == dtype
    dy = bf16_randn((M, N), seed=seed + 2).to(dtype).cuda()
    out.backward(dy)
    torch.cuda.synchronize()
    af, bf_, dyf = to_f32_np(a), to_f32_np(b), to_f32_np(dy)
    ref_out = OG.grouped_gemm_dequantized(af, bf_, lens, trans_b=True)
    ref_da = OG.grouped_gemm_dequantized(dyf, bf_, lens, trans_b=False)
    ref_db = OG.grouped_gemm_variable_k_dequantized(af, dyf, lens).transpose(0, 2, 1)  # [G, N, K]
    return a, b, gl, out, (ref_out, ref_da, ref_db)


SNR_GATE = 8.0  # E2M1 has one mantissa bit: the reference's bar for "correct layout"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kind,G_,M,N,K", [("zipf", 8, 4096, 1024, 1536), ("ragged", 4, 1000, 1408, 2048),
                                           ("balanced", 2, 256, 96, 160), ("ragged", 8, 2048, 288, 256)])
def test_grouped_gemm_fp4_autograd(dtype, kind, G_, M, N, K):
    lens = group_lens(kind, G_, M, 69)
    a, b, gl, out, (ref_out, ref_da, ref_db) = _autograd_case(lens, N, K, dtype, 70)
    assert OG.snr_db(ref_out, to_f32_np(out)) > SNR_GATE
    assert OG.snr_db(ref_da, to_f32_np(a.grad)) > SNR_GATE
    assert OG.snr_db(ref_db, to_f32_np(b.grad)) > SNR_GATE
    with torch.no_grad():
        out2 = turbo.ops.grouped_gemm_fp4(a, b, gl, trans_b=True, config=Float4QuantConfig())
    assert torch.equal(out2, out)


@pytest.mark.parametrize("lens,N,K", [((2048, 2048, 0, 0, 0, 0, 0, 0), 1024, 512), ((0, 1, 255, 257, 511, 513), 256, 256)],
                         ids=["empty-experts", "k256-zero-even-odd"])
def test_grouped_gemm_fp4_empty_and_odd_groups(lens, N, K):
    lens = np.asarray(lens, dtype=np.int64)
    a, b, gl, out, (ref_out, ref_da, ref_db) = _autograd_case(lens, N, K, torch.bfloat16, 73)
    assert OG.snr_db(ref_out, to_f32_np(out)) > SNR_GATE
    assert OG.snr_db(ref_da, to_f32_np(a.grad)) > SNR_GATE
    for g in range(len(lens)):
        if lens[g] == 0:
            assert torch.count_nonzero(b.grad[g]).item() == 0
        elif lens[g] >= 32:
            assert OG.snr_db(ref_db[g], to_f32_np(b.grad[g])) > SNR_GATE


@pytest.mark.parametrize("main_dtype", [torch.float32, torch.bfloat16])
def test_grouped_gemm_fp4_fused_grad_accum(main_dtype):
    """``fuse_bgrad_accum_pattern="megatron"`` leaves ``main_grad`` = previous + wgrad."""
    lens = group_lens("ragged", 4, 1024, 76)
    gl, _ = _offs(lens)
    a = bf16_randn((1024, 512), seed=77).cuda().requires_grad_(True)
    b = bf16_randn((4, 768, 512), seed=78).cuda().requires_grad_(True)
    dy = bf16_randn((1024, 768), seed=79).cuda()
    turbo.ops.grouped_gemm_fp4(a, b, gl).backward(dy)
    plain = b.grad.clone()
    b.grad = None
    b.main_grad = torch.full((4, 768, 512), 0.5, dtype=main_dtype, device="cuda")
    b.grad_added_to_main_grad = False
    turbo.ops.grouped_gemm_fp4(a, b, gl, fuse_bgrad_accum_pattern="megatron").backward(dy)
    torch.cuda.synchronize()
    assert b.grad_added_to_main_grad
    want = plain.float() + 0.5
    tol = 2e-2 * float(want.abs().max()) if main_dtype == torch.bfloat16 else 1e-2 * float(plain.float().abs().max())
    assert torch.allclose(b.main_grad.float(), want, rtol=0, atol=tol)


def test_grouped_quantize_fp4_ops_surface():
    lens = group_lens("ragged", 4, 600, 80)
    gl, offs = _offs(lens)
    x = bf16_randn((600, 256), seed=81).cuda()
    q, s, lp, op = turbo.ops.grouped_quantize_fp4(x, FP4, G.MX_BLOCKWISE, gl, offs, block_size=32, axis=1)
    assert torch.equal(lp, gl) and torch.equal(op, offs)
    y = turbo.ops.grouped_dequantize_fp4(q, torch.float32, G.MX_BLOCKWISE, block_size=32, axis=1, scale_inv=s)
    assert y.shape == (600, 256) and OG.snr_db(to_f32_np(x), to_f32_np(y)) > SNR_GATE
    out = turbo.ops.grouped_quantize_fp4_with_trans(x, FP4, G.MX_BLOCKWISE, gl, offs, block_size=32)
    assert len(out) == 8 and torch.equal(out[0].view(torch.uint8), q.view(torch.uint8))
    qc, sc, lc, oc = turbo.ops.grouped_quantize_fp4(x, FP4, G.MX_BLOCKWISE, gl, offs, block_size=32, axis=0)
    mc = int(oc[-1])  # what lies beyond the last padded group is unspecified
    assert torch.equal(out[7], oc) and torch.equal(out[2].view(torch.uint8)[:, : mc // 2], qc.view(torch.uint8)[:, : mc // 2])
    assert int(oc[-1]) % 256 == 0 and bool((lc % 256 == 0).all())
    with pytest.raises(NotImplementedError):  # the Hadamard transform is not combined with 2-D blocks
        turbo.ops.grouped_quantize_fp4(x, FP4, G.MX_BLOCKWISE, gl, offs, block_size=32, axis=1,
                                       scaling_recipe=ScalingRecipe(use_2d_block=True, use_rht=True))


@pytest.mark.parametrize("kind,G_,M,N", [("ragged", 8, 1000, 384), ("zeros", 8, 640, 128), ("zipf", 32, 4096, 512),
                                         ("ragged", 3, 77, 96)])
def test_grouped_mxfp4_quantizer_hadamard_bit_exact(kind, G_, M, N):
    """The recipe's Hadamard transform in the grouped quantizer (column direction = the wgrad
    operand, also the row direction) bit for bit against the oracle."""
    lens = group_lens(kind, G_, M, 82)
    gl, offs = _offs(lens)
    x = bf16_randn((M, N), seed=83, outlier_frac=0.002)
    rq, rs, cq, cs, _, _, _, ocol = qimpl.grouped_quantize_mxfp4_impl(
        x.cuda(), FP4, None, 32, gl, offs, with_trans=True, scaling_recipe=ScalingRecipe(),
        scaling_recipe_for_trans=ScalingRecipe(use_rht=True))
    o = Q.mx_grouped_quant(x.float().numpy(), lens, "e2m1", row_align=1, col_align=256, col_rht=True)
    mc = int(o["col_offs"][-1])
    assert np.array_equal(codes_np(rq), o["row"]) and np.array_equal(codes_np(rs), o["row_scale"])
    assert np.array_equal(codes_np(cq)[:, : mc // 2], o["col"]) and np.array_equal(codes_np(cs)[:, : mc // 32], o["col_scale"])
    q1, s1, _, _ = qimpl.grouped_quantize_mxfp4_impl(x.cuda(), FP4, 1, 32, gl, offs, scaling_recipe=ScalingRecipe(use_rht=True))
    o1 = Q.mx_grouped_quant(x.float().numpy(), lens, "e2m1", row_align=1, col_align=256, row_rht=True)
    assert np.array_equal(codes_np(q1), o1["row"]) and np.array_equal(codes_np(s1), o1["row_scale"])


def test_grouped_mxfp4_hadamard_cancels_in_wgrad():
    """Both wgrad operands carry the transform along the token axis: the variable-K product of the
    transformed quantizations estimates the same dW as the plain ones, at least as well."""
    lens = group_lens("ragged", 4, 2048, 84)
    gl, offs = _offs(lens)
    x = bf16_randn((2048, 512), seed=85, outlier_frac=0.01)
    dy = bf16_randn((2048, 384), seed=86, outlier_frac=0.01)
    ref = OG.grouped_gemm_variable_k_dequantized(x.float().numpy(), dy.float().numpy(), lens).transpose(0, 2, 1)
    snr = {}
    for rht in (False, True):
        rec = ScalingRecipe(use_rht=rht)
        xq, xs, lc, ocol = qimpl.grouped_quantize_mxfp4_impl(x.cuda(), FP4, 0, 32, gl, offs, scaling_recipe=rec)
        gq, gs, _, _ = qimpl.grouped_quantize_mxfp4_impl(dy.cuda(), FP4, 0, 32, gl, offs, scaling_recipe=rec)
        out = gimpl.grouped_gemm_fp4_variable_k_impl(gq, xq, gs, xs, lc, ocol, False, False, False, torch.float32,
                                                     G.MX_BLOCKWISE.value, None, 0)
        snr[rht] = OG.snr_db(ref, to_f32_np(out))
    assert snr[True] > SNR_GATE and snr[True] > snr[False] - 1.0, snr


@pytest.mark.parametrize("grouped", [True, False])
def test_fp4_gradient_stochastic_rounding(grouped):
    """``Float4QuantConfig(use_gradient_sr=True)``: forward is unchanged, the gradients pass the same
    SNR gate, and two backward passes differ (the gradient quantizers draw a fresh seed)."""
    lens = group_lens("ragged", 4, 1024, 87)
    gl, _ = _offs(lens)
    a = bf16_randn((1024, 512), seed=88).cuda().requires_grad_(True)
    b = (bf16_randn((4, 384, 512), seed=89) if grouped else bf16_randn((384, 512), seed=89)).cuda().requires_grad_(True)
    dy = bf16_randn((1024, 384), seed=90).cuda()
    cfg, cfg_sr = Float4QuantConfig(), Float4QuantConfig(use_gradient_sr=True)

    def run(c):
        a.grad = b.grad = None
        y = turbo.ops.grouped_gemm_fp4(a, b, gl, config=c) if grouped else turbo.ops.gemm_fp4(a, b, trans_b=True, config=c)
        y.backward(dy)
        return y.detach().clone(), a.grad.clone(), b.grad.clone()

    y0, da0, db0 = run(cfg)
    y1, da1, db1 = run(cfg_sr)
    y2, da2, db2 = run(cfg_sr)
    assert torch.equal(y0, y1) and torch.equal(y1, y2)
    assert not torch.equal(da1, da2) and not torch.equal(db1, db2)
    af, bf_, dyf = to_f32_np(a), to_f32_np(b), to_f32_np(dy)
    if grouped:
        ref_da = OG.grouped_gemm_dequantized(dyf, bf_, lens, trans_b=False)
        ref_db = OG.grouped_gemm_variable_k_dequantized(af, dyf, lens).transpose(0, 2, 1)
    else:
        ref_da, ref_db = dyf @ bf_, dyf.T @ af
    for da, db in ((da1, db1), (da2, db2)):
        assert OG.snr_db(ref_da, to_f32_np(da)) > SNR_GATE and OG.snr_db(ref_db, to_f32_np(db)) > SNR_GATE
