"""GPU parity of the grouped MXFP8 path (MoE experts with E8M0 block scales): the grouped quantizer
(rows of every group padded to 32 for the row direction, to 128 for the transposed column
direction) bit for bit against the oracle, the row-group GEMM (padded A rows, tightly packed
output) and the variable-K wgrad GEMM against the fp32 matmul of the de-quantized operands
(max |err| / max |ref| <= 1e-2, cosine >= 0.9999), and the autograd op at the reference's SNR gate
(tests/pytorch/ops/test_grouped_gemm_fp8.py of the reference: 25 dB E4M3, 20 dB E5M2 / HYBRID)."""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, codes_np, gemm_gate, group_lens, to_f32_np
from oracle import gemm as OG
from oracle import quantize as Q

pytestmark = pytest.mark.gpu

FMT = {torch.float8_e4m3fn: "e4m3", torch.float8_e5m2: "e5m2"}


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, Float8QuantConfig, Format, ScaleDtype, ScalingRecipe, gimpl, qimpl
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, Format, ScaleDtype, ScalingRecipe
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.kernels.grouped_gemm import grouped_gemm_fp8_impl as gimpl
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qimpl


def _gate(ref, got, what=""):
    return gemm_gate(ref, got, what)


def _offs(lens):
    gl = torch.from_numpy(lens).cuda()
    return gl, torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)


QCASES = [("balanced", 4, 512, 256), ("ragged", 8, 1000, 384), ("zeros", 8, 640, 128), ("zipf", 32, 4096, 512),
          ("ragged", 3, 77, 96), ("balanced", 1, 200, 160)]


@pytest.mark.parametrize("kind,G_,M,N", QCASES)
@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_grouped_mx_quantizer_bit_exact(kind, G_, M, N, dtype):
    lens = group_lens(kind, G_, M, 41)
    gl, offs = _offs(lens)
    x = bf16_randn((M, N), seed=42, outlier_frac=0.002)
    rq, rs, cq, cs, lr, orow, lc, ocol = qimpl.grouped_quantize_mxfp8_impl(x.cuda(), dtype, None, 32, gl, offs, with_trans=True)
    o = Q.mx_grouped_quant(x.float().numpy(), lens, FMT[dtype])
    G1 = G_ * 32, G_ * 128
    assert rq.shape == (-(-(M + G1[0]) // 32) * 32, -(-N // 128) * 128) and cq.shape == (N, -(-(M + G1[1]) // 128) * 128)
    assert np.array_equal(lr.cpu().numpy(), o["row_lens"]) and np.array_equal(orow.cpu().numpy(), o["row_offs"])
    assert np.array_equal(lc.cpu().numpy(), o["col_lens"]) and np.array_equal(ocol.cpu().numpy(), o["col_offs"])
    mr, mc = int(o["row_offs"][-1]), int(o["col_offs"][-1])
    assert np.array_equal(codes_np(rq)[:mr], o["row"]) and np.array_equal(codes_np(rs)[:mr], o["row_scale"])
    assert np.array_equal(codes_np(cq)[:, :mc], o["col"]) and np.array_equal(codes_np(cs)[:, : mc // 32], o["col_scale"])
    # one direction at a time gives the same tensors
    q1, s1, l1, o1 = qimpl.grouped_quantize_mxfp8_impl(x.cuda(), dtype, 1, 32, gl, offs)
    q0, s0, l0, o0 = qimpl.grouped_quantize_mxfp8_impl(x.cuda(), dtype, 0, 32, gl, offs)
    assert np.array_equal(codes_np(q1)[:mr], o["row"]) and np.array_equal(codes_np(s1)[:mr], o["row_scale"])
    assert np.array_equal(codes_np(q0)[:, :mc], o["col"]) and np.array_equal(codes_np(s0)[:, : mc // 32], o["col_scale"])
    assert torch.equal(o1, orow) and torch.equal(o0, ocol) and torch.equal(l1, lr) and torch.equal(l0, lc)
    # the de-quantizer gathers the packed rows back
    for axis, (q, s, op) in ((1, (rq, rs, orow)), (0, (cq, cs, ocol))):
        y = qimpl.grouped_dequantize_mxfp8_impl(q, torch.float32, axis, 32, s, offs, op, total_M=M)
        if axis == 1:
            ref = Q.mx_dequant(o["row"], o["row_scale"], FMT[dtype])
            pad_offs = o["row_offs"]
        else:
            ref = Q.mx_dequant(o["col"], o["col_scale"], FMT[dtype]).T
            pad_offs = o["col_offs"]
        starts = np.concatenate([[0], np.cumsum(lens)])
        want = np.concatenate([ref[pad_offs[g] : pad_offs[g] + lens[g]] for g in range(G_)], axis=0)
        assert y.shape[0] == M and np.array_equal(to_f32_np(y)[:, : want.shape[1]], want), f"axis {axis}"
        del starts


@pytest.mark.parametrize("kind,G_,M,N", [("ragged", 8, 1000, 384), ("zeros", 8, 640, 128), ("zipf", 32, 4096, 512), ("ragged", 3, 77, 96)])
@pytest.mark.parametrize("row_2d,col_2d", [(True, True), (True, False), (False, True)])
def test_grouped_mx_quantizer_2d_blocks_bit_exact(kind, G_, M, N, row_2d, col_2d):
    """32 x 32 blocks in the grouped quantizer: counted from each group's first row (the rows
    behind a group's end are zeros), one exponent replicated into the scale slot of each row."""
    lens = group_lens(kind, G_, M, 51)
    gl, offs = _offs(lens)
    x = bf16_randn((M, N), seed=52, outlier_frac=0.002)
    dtype = torch.float8_e4m3fn
    rq, rs, cq, cs, lr, orow, lc, ocol = qimpl.grouped_quantize_mxfp8_impl(
        x.cuda(), dtype, None, 32, gl, offs, with_trans=True, scaling_recipe=ScalingRecipe(use_2d_block=row_2d),
        scaling_recipe_for_trans=ScalingRecipe(use_2d_block=col_2d))
    o = Q.mx_grouped_quant(x.float().numpy(), lens, "e4m3", row_2d=row_2d, col_2d=col_2d)
    mr, mc = int(o["row_offs"][-1]), int(o["col_offs"][-1])
    assert np.array_equal(codes_np(rs)[:mr], o["row_scale"]) and np.array_equal(codes_np(rq)[:mr], o["row"])
    assert np.array_equal(codes_np(cs)[:, : mc // 32], o["col_scale"]) and np.array_equal(codes_np(cq)[:, :mc], o["col"])
    # one direction alone gives the same tensors
    q1, s1, _, _ = qimpl.grouped_quantize_mxfp8_impl(x.cuda(), dtype, 1, 32, gl, offs, scaling_recipe=ScalingRecipe(use_2d_block=row_2d))
    q0, s0, _, _ = qimpl.grouped_quantize_mxfp8_impl(x.cuda(), dtype, 0, 32, gl, offs, scaling_recipe=ScalingRecipe(use_2d_block=col_2d))
    assert np.array_equal(codes_np(q1)[:mr], o["row"]) and np.array_equal(codes_np(s1)[:mr], o["row_scale"])
    assert np.array_equal(codes_np(q0)[:, :mc], o["col"]) and np.array_equal(codes_np(s0)[:, : mc // 32], o["col_scale"])


def test_grouped_mx_quantizer_shuffled_outputs():
    """``shuffle_out`` / ``shuffle_scale`` in the grouped quantizer: the pre-shuffled forms of the
    plain outputs (the same pass as behind the dense quantizers), undone by the inverse ops."""
    lens = group_lens("ragged", 8, 1000, 53)
    gl, offs = _offs(lens)
    x = bf16_randn((1000, 384), seed=54).cuda()
    dtype = torch.float8_e4m3fn
    plain = qimpl.grouped_quantize_mxfp8_impl(x, dtype, None, 32, gl, offs, with_trans=True)
    rec = ScalingRecipe(shuffle_scale=True, shuffle_out=True)
    shuf = qimpl.grouped_quantize_mxfp8_impl(x, dtype, None, 32, gl, offs, with_trans=True, scaling_recipe=rec,
                                             scaling_recipe_for_trans=rec)
    mr, mc = int(plain[5][-1]), int(plain[7][-1])
    for qi_, si_, rows in ((0, 1, mr), (2, 3, 384)):
        q, s = shuf[qi_], shuf[si_]
        assert q.shape == plain[qi_].shape and s.shape[0] % 256 == 0 and s.shape[1] % 8 == 0
        assert not torch.equal(q.view(torch.uint8), plain[qi_].view(torch.uint8))
        back, sback = qimpl.mx_plain_layout(q, s, True, True)
        back = back.view(torch.uint8)
        if qi_ == 0:
            assert torch.equal(back[:rows], plain[0].view(torch.uint8)[:rows])
            assert torch.equal(sback.view(torch.uint8)[:rows], plain[1].view(torch.uint8)[:rows])
        else:
            assert torch.equal(back[:, :mc], plain[2].view(torch.uint8)[:, :mc])
            assert torch.equal(sback.view(torch.uint8)[:, : mc // 32], plain[3].view(torch.uint8)[:, : mc // 32])
    assert all(torch.equal(a, b) for a, b in zip(shuf[4:], plain[4:]))


GCASES = [("balanced", 4, 1024, 512, 512), ("ragged", 8, 3000, 384, 1024), ("zeros", 8, 2048, 256, 512),
          ("zipf", 32, 8192, 1024, 768), ("ragged", 3, 77, 96, 640), ("zipf", 16, 4096, 2048, 512),
          # K below four 128-byte slabs, and K that the quantizer pads to the next multiple of 128
          ("ragged", 4, 600, 256, 128), ("zipf", 8, 1024, 384, 256), ("balanced", 2, 256, 128, 384), ("ragged", 3, 300, 256, 160)]


@pytest.mark.parametrize("kind,G_,M,N,K", GCASES)
@pytest.mark.parametrize("fa,fb", [(torch.float8_e4m3fn, torch.float8_e4m3fn), (torch.float8_e5m2, torch.float8_e4m3fn)])
def test_grouped_mx_forward_product(kind, G_, M, N, K, fa, fb):
    lens = group_lens(kind, G_, M, 43)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=44)
    w = bf16_randn((G_, N, K), seed=45)
    rq, rs, lr, orow = qimpl.grouped_quantize_mxfp8_impl(x.cuda(), fa, 1, 32, gl, offs)
    wq, ws = qimpl.quantize_mxfp8_impl(w.cuda(), fb, 2, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))
    out = gimpl.grouped_gemm_fp8_impl(rq, wq, rs, ws, gl, orow, False, True, torch.bfloat16, G.MX_BLOCKWISE.value, None, 0,
                                      False, offs)
    torch.cuda.synchronize()
    assert out.shape == (rq.shape[0], N)
    o = Q.mx_grouped_quant(x.float().numpy(), lens, FMT[fa])
    a_pad = Q.mx_dequant(o["row"], o["row_scale"], FMT[fa])[:, :K]
    a_deq = np.concatenate([a_pad[o["row_offs"][g] : o["row_offs"][g] + lens[g]] for g in range(G_)], axis=0)
    w_deq = np.stack([Q.mx_dequant(codes_np(wq[g]), codes_np(ws[g]), FMT[fb])[:, :K] for g in range(G_)])
    ref = OG.grouped_gemm_dequantized(a_deq, w_deq, lens, trans_b=True)
    _gate(ref, to_f32_np(out[:M]), f"{kind} G={G_} {M}x{N}x{K}")
    assert not bool(out[M:].float().abs().max() > 0) if out.shape[0] > M else True
    # the dense (unpadded) row layout with one set of offsets gives the same rows
    dq, dsc = qimpl.quantize_mxfp8_impl(x.cuda(), fa, 1, 32)
    out2 = gimpl.grouped_gemm_fp8_impl(dq, wq, dsc, ws, gl, offs, False, True, torch.bfloat16, G.MX_BLOCKWISE.value, None, 0)
    assert torch.equal(out2[:M], out[:M])


@pytest.mark.parametrize("kind,G_,M,N,K", [("zipf", 32, 8192, 1024, 768), ("ragged", 8, 3000, 384, 1024), ("zeros", 8, 2048, 256, 512),
                                           ("ragged", 3, 77, 96, 640), ("zipf", 16, 4096, 2048, 2048)])
@pytest.mark.parametrize("padded", [False, True])
def test_grouped_mx_eight_wavefront_tile(kind, G_, M, N, K, padded):
    """tile_cfg 4 (256 x 256 tile, eight wavefronts, gemm_mx8.h with row groups) gives the bits of
    the automatic configuration: the same products added in the same order, with the per-group
    padded row layout of the grouped quantizer and with the tight one."""
    lens = group_lens(kind, G_, M, 143)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=144).cuda()
    w = bf16_randn((G_, N, K), seed=145).cuda()
    wq, ws = qimpl.quantize_mxfp8_impl(w, torch.float8_e4m3fn, 2, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))
    if padded:
        rq, rs, _, orow = qimpl.grouped_quantize_mxfp8_impl(x, torch.float8_e4m3fn, 1, 32, gl, offs)
        run = lambda: gimpl.grouped_gemm_fp8_impl(rq, wq, rs, ws, gl, orow, False, True, torch.bfloat16, G.MX_BLOCKWISE.value,  # noqa: E731
                                                  None, 0, False, offs)
    else:
        rq, rs = qimpl.quantize_mxfp8_impl(x, torch.float8_e4m3fn, 1, 32)
        run = lambda: gimpl.grouped_gemm_fp8_impl(rq, wq, rs, ws, gl, offs, False, True, torch.bfloat16, G.MX_BLOCKWISE.value,  # noqa: E731
                                                  None, 0)
    auto = run()
    gimpl.MX_TILE_CFG = 4
    try:
        got = run()
    finally:
        gimpl.MX_TILE_CFG = 0
    torch.cuda.synchronize()
    assert torch.equal(got, auto)


@pytest.mark.parametrize("kind,G_,M,N,K", GCASES)
@pytest.mark.parametrize("trans_c", [False, True])
def test_grouped_mx_variable_k_product(kind, G_, M, N, K, trans_c):
    lens = group_lens(kind, G_, M, 46)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=47)
    dy = bf16_randn((M, N), seed=48)
    xq, xs, lc, ocol = qimpl.grouped_quantize_mxfp8_impl(x.cuda(), torch.float8_e4m3fn, 0, 32, gl, offs)
    gq, gs, _, _ = qimpl.grouped_quantize_mxfp8_impl(dy.cuda(), torch.float8_e5m2, 0, 32, gl, offs)
    out = gimpl.grouped_gemm_fp8_variable_k_impl(gq, xq, gs, xs, lc, ocol, False, False, trans_c, torch.float32,
                                                 G.MX_BLOCKWISE.value, None, 0)
    torch.cuda.synchronize()
    assert out.shape == ((G_, K, N) if trans_c else (G_, N, K))
    ox = Q.mx_grouped_quant(x.float().numpy(), lens, "e4m3")
    og = Q.mx_grouped_quant(dy.float().numpy(), lens, "e5m2")
    xd = Q.mx_dequant(ox["col"], ox["col_scale"], "e4m3")  # [K, Mc]
    gd = Q.mx_dequant(og["col"], og["col_scale"], "e5m2")  # [N, Mc]
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
    gimpl.grouped_gemm_fp8_variable_k_accum_impl(gq, xq, gs, xs, lc, ocol, False, False, trans_c, torch.float32,
                                                 G.MX_BLOCKWISE.value, None, 0, acc)
    assert torch.allclose(acc, out + 1, rtol=0, atol=1e-3 * float(out.abs().max()) + 1e-6)


@pytest.mark.parametrize("fmt,gate", [("E4M3", 25), ("E5M2", 20), ("HYBRID", 20)])
@pytest.mark.parametrize("kind,G_,M,N,K", [("zipf", 8, 4096, 1024, 512), ("ragged", 4, 1000, 512, 1024),
                                           ("ragged", 4, 1000, 256, 128), ("zipf", 8, 2048, 128, 384)])
def test_grouped_gemm_fp8_mx_autograd(fmt, gate, kind, G_, M, N, K):
    """The MX_BLOCKWISE op end to end (grouped quantizers, forward, dgrad, wgrad) against the
    unquantized grouped matmul; empty experts get a zero weight gradient; a forward-only call
    gives the same output."""
    lens = group_lens(kind, G_, M, 49)
    gl, _ = _offs(lens)
    a = bf16_randn((M, K), seed=50).cuda().requires_grad_(True)
    b = bf16_randn((G_, N, K), seed=51).cuda().requires_grad_(True)
    cfg = Float8QuantConfig(format=getattr(Format, fmt), granularity=G.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0)
    out = turbo.ops.grouped_gemm_fp8(a, b, gl, trans_b=True, config=cfg)
    assert out.shape == (M, N) and out.dtype == torch.bfloat16
    dy = bf16_randn((M, N), seed=52).cuda()
    out.backward(dy)
    torch.cuda.synchronize()
    af, bf_, dyf = to_f32_np(a), to_f32_np(b), to_f32_np(dy)
    ref_out = OG.grouped_gemm_dequantized(af, bf_, lens, trans_b=True)
    ref_da = OG.grouped_gemm_dequantized(dyf, bf_, lens, trans_b=False)
    ref_db = OG.grouped_gemm_variable_k_dequantized(af, dyf, lens).transpose(0, 2, 1)  # [G, N, K]
    assert OG.snr_db(ref_out, to_f32_np(out)) > gate
    assert OG.snr_db(ref_da, to_f32_np(a.grad)) > gate
    assert OG.snr_db(ref_db, to_f32_np(b.grad)) > gate
    for g in range(G_):
        if lens[g] == 0:
            assert torch.count_nonzero(b.grad[g]).item() == 0
    with torch.no_grad():
        out2 = turbo.ops.grouped_gemm_fp8(a, b, gl, trans_b=True, config=cfg)
    assert torch.equal(out2, out)


def test_grouped_quantize_fp8_ops_surface():
    """``grouped_quantize_fp8`` / ``..._with_trans`` / ``grouped_dequantize_fp8`` of the op layer."""
    lens = group_lens("ragged", 4, 600, 53)
    gl, offs = _offs(lens)
    x = bf16_randn((600, 256), seed=54).cuda()
    q, s, lp, op = turbo.ops.grouped_quantize_fp8(x, turbo.float8_e4m3, G.MX_BLOCKWISE, gl, offs, block_size=32, axis=-1)
    y = turbo.ops.grouped_dequantize_fp8(q, torch.float32, G.MX_BLOCKWISE, offs, op, block_size=32, axis=1, scale_inv=s,
                                         total_M=600)
    assert y.shape == (600, 256)
    assert OG.snr_db(to_f32_np(x), to_f32_np(y)) > 25
    out = turbo.ops.grouped_quantize_fp8_with_trans(x, turbo.float8_e4m3, G.MX_BLOCKWISE, gl, offs, block_size=32)
    assert len(out) == 8 and torch.equal(out[0][: int(op[-1])], q[: int(op[-1])]) and torch.equal(out[5], op)
    yc = turbo.ops.grouped_dequantize_fp8(out[2], torch.float32, G.MX_BLOCKWISE, offs, out[7], block_size=32, axis=0,
                                          scale_inv=out[3], total_M=600)
    assert OG.snr_db(to_f32_np(x), to_f32_np(yc)[:, :256]) > 25
