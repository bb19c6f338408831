"""GPU checks at the full shapes of the benchmark configurations, through properties that do not
need a CPU matmul of the whole problem:

* sampled outputs against float64 dot products of the de-quantized operands (oracle
  de-quantizers), same gate as everywhere: max |err| / max |ref| <= 1e-2, cosine >= 0.9999;
* exact invariances of a scaled GEMM: doubling a scale vector doubles the bf16 output bit for bit,
  permuting the rows of A permutes the rows of C, a column slice of B gives the column slice of C,
  an E8M0 byte raised by one doubles the MX product;
* quantizers at full size: bytes and scales of sampled rows / tiles bit-exact against the oracle,
  round-trip error within one quantization step of the block's scale.
"""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, codes_np, gemm_gate, group_lens, to_f32_np
from oracle import gemm as OG
from oracle import quantize as Q

pytestmark = pytest.mark.gpu

FP4 = getattr(torch, "float4_e2m1fn_x2", None)


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, ScalingRecipe, gi, g4, gg, qi
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.core.low_precision import ScalingRecipe
    from primus_turbo.pytorch.kernels.gemm import gemm_fp4_impl as g4
    from primus_turbo.pytorch.kernels.gemm import gemm_fp8_impl as gi
    from primus_turbo.pytorch.kernels.grouped_gemm import grouped_gemm_fp8_impl as gg
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi


def _sampled_gate(out, a_deq_rows, b_deq_rows, rows, cols, what):
    """out[rows][:, cols] against float64 dot products of the given de-quantized rows."""
    ref = a_deq_rows.astype(np.float64) @ b_deq_rows.astype(np.float64).T
    got = to_f32_np(out[torch.as_tensor(rows)][:, torch.as_tensor(cols)])
    ref = torch.from_numpy(ref.astype(np.float32)).to(out.dtype).float().numpy()
    gemm_gate(ref, got, what)  # cosine, range-relative maximum, Frobenius-relative error, element-wise bound


def _pick(n, k, seed):
    return np.sort(np.random.default_rng(seed).choice(n, size=k, replace=False))


def test_rowwise_gemm_8192_samples_and_invariances():
    M = N = K = 8192
    a = bf16_randn((M, K), seed=201, scale=0.02).cuda()
    b = bf16_randn((N, K), seed=202, scale=0.02).cuda()
    aq, asi = turbo.ops.quantize_fp8(a, turbo.float8_e4m3, G.ROWWISE, axis=-1)
    bq, bsi = turbo.ops.quantize_fp8(b, turbo.float8_e4m3, G.ROWWISE, axis=-1)
    out = gi.gemm_fp8_impl(aq, asi, False, bq, bsi, True, torch.bfloat16, False, G.ROWWISE.value, 0)
    rows, cols = _pick(M, 96, 1), _pick(N, 128, 2)
    a_deq = Q.fp8_dequant(codes_np(aq)[rows], to_f32_np(asi)[rows], "e4m3")
    b_deq = Q.fp8_dequant(codes_np(bq)[cols], to_f32_np(bsi)[cols], "e4m3")
    _sampled_gate(out, a_deq, b_deq, rows, cols, "rowwise 8192^3")
    # scale linearity (exact: a power of two commutes with every rounding involved)
    out2 = gi.gemm_fp8_impl(aq, asi * 2, False, bq, bsi, True, torch.bfloat16, False, G.ROWWISE.value, 0)
    assert torch.equal(out2, out * 2)
    # row permutation of A
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(3)).cuda()
    outp = gi.gemm_fp8_impl(aq[perm].contiguous(), asi[perm].contiguous(), False, bq, bsi, True, torch.bfloat16, False,
                            G.ROWWISE.value, 0)
    assert torch.equal(outp, out[perm])
    # column slice of B
    outs = gi.gemm_fp8_impl(aq, asi, False, bq[: N // 2].contiguous(), bsi[: N // 2].contiguous(), True, torch.bfloat16,
                            False, G.ROWWISE.value, 0)
    assert torch.equal(outs, out[:, : N // 2])


@pytest.mark.parametrize("M,N,K", [(16384, 7168, 2048), (16384, 4096, 7168), (8192, 8192, 8192)])
def test_blockwise_gemm_full_shapes(M, N, K):
    a = bf16_randn((M, K), seed=203).cuda()
    w = bf16_randn((N, K), seed=204).cuda()
    aq, asi = qi.quant_fp8_blockwise_impl(a, torch.float8_e4m3fn, -1, 128)
    wq, wsi = qi.quant_fp8_blockwise_for_weight_impl(w, torch.float8_e4m3fn, 128)
    out = gi.gemm_fp8_impl(aq, asi, False, wq, wsi, True, torch.bfloat16, False, G.BLOCKWISE.value, 0)
    rows = _pick(M, 96, 4)
    cols = np.arange(256, 512)  # two whole weight tiles
    a_deq = Q.fp8_blockwise_dequant(codes_np(aq)[rows], to_f32_np(asi)[rows], 1, "e4m3", 128)
    w_deq = Q.fp8_blockwise_weight_dequant(codes_np(wq)[256:512], to_f32_np(wsi)[2:4], "e4m3", 128)
    _sampled_gate(out, a_deq, w_deq, rows, cols, f"blockwise {M}x{N}x{K}")
    out2 = gi.gemm_fp8_impl(aq, asi * 2, False, wq, wsi * 0.5, True, torch.bfloat16, False, G.BLOCKWISE.value, 0)
    assert torch.equal(out2, out)  # the factors cancel exactly in every K block
    perm = torch.randperm(M, generator=torch.Generator().manual_seed(5)).cuda()
    outp = gi.gemm_fp8_impl(aq[perm].contiguous(), asi[perm].contiguous(), False, wq, wsi, True, torch.bfloat16, False,
                            G.BLOCKWISE.value, 0)
    assert torch.equal(outp, out[perm])


@pytest.mark.parametrize("fp4", [False, True])
@pytest.mark.parametrize("M,N,K", [(16384, 16384, 16384), (8192, 28672, 8192)])
def test_mx_gemm_full_shapes(fp4, M, N, K):
    if fp4 and FP4 is None:
        pytest.skip("torch has no float4_e2m1fn_x2")
    fmt = "e2m1" if fp4 else "e4m3"
    quant = qi.quantize_mxfp4_impl if fp4 else qi.quantize_mxfp8_impl
    qdt = FP4 if fp4 else torch.float8_e4m3fn
    a = bf16_randn((M, K), seed=205).cuda()
    b = bf16_randn((N, K), seed=206).cuda()
    aq, as_ = quant(a, qdt, 1, 32)
    bq, bs = quant(b, qdt, 1, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))
    del a, b

    def mm(sa):
        if fp4:
            return g4.gemm_fp4_impl(aq, sa, False, bq, bs, True, torch.bfloat16, False, G.MX_BLOCKWISE.value, 0)
        return gi.gemm_fp8_impl(aq, sa, False, bq, bs, True, torch.bfloat16, False, G.MX_BLOCKWISE.value, 0)

    out = mm(as_)
    rows, cols = _pick(M, 64, 6), _pick(N, 128, 7)
    a_deq = Q.mx_dequant(codes_np(aq)[rows], codes_np(as_)[rows], fmt)
    b_deq = Q.mx_dequant(codes_np(bq)[cols], codes_np(bs)[cols], fmt)
    _sampled_gate(out, a_deq, b_deq, rows, cols, f"mx {fmt} {M}x{N}x{K}")
    # every E8M0 byte of A raised by one: the product doubles exactly
    as2 = (as_.view(torch.uint8) + 1).view(as_.dtype)
    assert torch.equal(mm(as2), out * 2)


@pytest.mark.parametrize("N,K", [(4096, 7168), (7168, 2048)])
def test_grouped_forward_full_config(N, K):
    Gn, M = 32, 32768
    lens = group_lens("zipf", Gn, M, 7)
    gl = torch.from_numpy(lens).cuda()
    offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)
    x = bf16_randn((M, K), seed=207).cuda()
    w = bf16_randn((Gn, N, K), seed=208).cuda()
    qr, _, sr, _, _, _ = qi.quant_fp8_blockwise_segment_m_row_col_impl(x, torch.float8_e4m3fn, 128, gl, offs, N)
    wq, ws = qi.quant_fp8_blockwise_for_weight_impl(w, torch.float8_e4m3fn, 128)
    out = gg.grouped_gemm_fp8_impl(qr, wq, sr, ws, gl, offs, False, True, torch.bfloat16, G.BLOCKWISE.value, None, 0)
    starts = np.concatenate([[0], np.cumsum(lens)])
    rng = np.random.default_rng(8)
    sr_t = np.ascontiguousarray(to_f32_np(sr).T)  # [M, K / 128]
    for g in [g for g in range(Gn) if lens[g] > 0][::5]:
        rows = np.sort(starts[g] + rng.choice(int(lens[g]), size=min(24, int(lens[g])), replace=False))
        a_deq = Q.fp8_blockwise_dequant(codes_np(qr)[rows], sr_t[rows], 1, "e4m3", 128)
        w_deq = Q.fp8_blockwise_weight_dequant(codes_np(wq[g])[128:384], to_f32_np(ws[g])[1:3], "e4m3", 128)
        _sampled_gate(out, a_deq, w_deq, rows, np.arange(128, 384), f"grouped expert {g}")
    # swapping two experts' weights and token blocks of equal length swaps their outputs: use the
    # self-consistency of one expert instead -- its rows alone, as a one-group problem
    g = int(np.argmax(lens))
    r0, r1 = int(starts[g]), int(starts[g + 1])
    one = torch.tensor([r1 - r0], dtype=torch.int64).cuda()
    one_offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(one)
    solo = gg.grouped_gemm_fp8_impl(qr[r0:r1].contiguous(), wq[g : g + 1].contiguous(), sr[:, r0:r1].contiguous(),
                                    ws[g : g + 1].contiguous(), one, one_offs, False, True, torch.bfloat16,
                                    G.BLOCKWISE.value, None, 0)
    assert torch.equal(solo, out[r0:r1])


@pytest.mark.parametrize("N,K", [(4096, 7168), (7168, 2048)])
def test_grouped_backward_full_config(N, K):
    """dgrad and variable-K wgrad of the MoE configuration at full size (32 experts, 32768 Zipf
    tokens, two experts empty), on the operands the autograd function hands them: sampled outputs
    of sampled experts against float64 dot products of the de-quantized operands; an expert
    without tokens gets an exactly zero weight gradient, and with beta = 1 its slice of the
    accumulation buffer stays untouched bit for bit."""
    Gn, M = 32, 32768
    f8 = torch.float8_e4m3fn
    lens = group_lens("zipf", Gn, M, 7)
    assert (lens == 0).sum() >= 2
    gl = torch.from_numpy(lens).cuda()
    offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)
    x = bf16_randn((M, K), seed=211).cuda()
    dy = bf16_randn((M, N), seed=212).cuda()
    w = bf16_randn((Gn, N, K), seed=213).cuda()
    _, x_col_t, _, x_scol, _, _ = qi.quant_fp8_blockwise_segment_m_row_col_t_impl(x, f8, 128, gl, offs)
    g_row, g_col_t, g_srow, g_scol, vk_lens, vk_offs = qi.quant_fp8_blockwise_segment_m_row_col_t_impl(dy, f8, 128, gl, offs)
    wq, wq_t, ws = qi.quant_fp8_blockwise_for_weight_dual_impl(w, f8, block_size=128)
    ws_t = ws.transpose(-2, -1).contiguous()
    del x, dy, w
    starts = np.concatenate([[0], np.cumsum(lens)])
    live = [g for g in range(Gn) if lens[g] > 0]
    empty = [g for g in range(Gn) if lens[g] == 0]
    rng = np.random.default_rng(9)

    # ---- dgrad: dX[rows of g] = dY_g . W_g   ([M, N] x [N, K] -> [M, K]) ----
    dx = gg.grouped_gemm_fp8_impl(g_row, wq_t, g_srow, ws_t, gl, offs, False, True, torch.bfloat16, G.BLOCKWISE.value, None, 0)
    assert tuple(dx.shape) == (M, K)
    gs_t = np.ascontiguousarray(to_f32_np(g_srow).T)  # [M, N / 128]
    for g in live[::5]:
        rows = np.sort(starts[g] + rng.choice(int(lens[g]), size=min(24, int(lens[g])), replace=False))
        a_deq = Q.fp8_blockwise_dequant(codes_np(g_row)[rows], gs_t[rows], 1, "e4m3", 128)
        # rows 128..383 of W_g^T [K, N] = output columns 128..383
        wt_deq = Q.fp8_blockwise_weight_dequant(codes_np(wq_t[g])[128:384], to_f32_np(ws_t[g])[1:3], "e4m3", 128)
        _sampled_gate(dx, a_deq, wt_deq, rows, np.arange(128, 384), f"dgrad expert {g}")

    # ---- wgrad: dW[g] = dY_g^T . X_g over the group's 128-padded token range ----
    dw = gg.grouped_gemm_fp8_variable_k_impl(x_col_t, g_col_t, x_scol, g_scol, vk_lens, vk_offs, False, True, True,
                                             torch.bfloat16, G.BLOCKWISE.value, None, 0)
    assert tuple(dw.shape) == (Gn, N, K)
    vo = vk_offs.cpu().numpy()
    xs_t = np.ascontiguousarray(to_f32_np(x_scol).T)  # [K, M_pad / 128]
    gsc_t = np.ascontiguousarray(to_f32_np(g_scol).T)  # [N, M_pad / 128]
    for g in empty:
        assert torch.count_nonzero(dw[g]).item() == 0, f"expert {g} has no tokens: its weight gradient must be exactly zero"
    ncols, krows = _pick(N, 48, 10), _pick(K, 40, 11)
    for g in (live[0], live[len(live) // 2], int(np.argmax(lens))):
        t0, t1 = int(vo[g]), int(vo[g + 1])
        gy = Q.fp8_blockwise_dequant(codes_np(g_col_t)[ncols][:, t0:t1], gsc_t[ncols][:, t0 // 128 : t1 // 128], 1, "e4m3", 128)
        gx = Q.fp8_blockwise_dequant(codes_np(x_col_t)[krows][:, t0:t1], xs_t[krows][:, t0 // 128 : t1 // 128], 1, "e4m3", 128)
        _sampled_gate(dw[g], gy, gx, ncols, krows, f"wgrad expert {g}")

    # ---- beta = 1: accumulate into an fp32 buffer; empty experts stay untouched ----
    base = torch.empty((Gn, N, K), dtype=torch.float32, device="cuda").normal_(generator=torch.Generator("cuda").manual_seed(3))
    keep = {g: base[g].clone() for g in empty}
    g_big = int(np.argmax(lens))
    before = base[g_big, :64].clone()
    gg.grouped_gemm_fp8_variable_k_accum_impl(x_col_t, g_col_t, x_scol, g_scol, vk_lens, vk_offs, False, True, True,
                                              torch.float32, G.BLOCKWISE.value, None, 0, base)
    for g in empty:
        assert torch.equal(base[g], keep[g]), f"beta = 1 touched the buffer of the empty expert {g}"
    added = (base[g_big, :64] - before).float()
    want = dw[g_big, :64].float()
    assert (added - want).abs().max().item() <= 2e-2 * want.abs().max().item()  # bf16 rounding of dw + fp32 cancellation


def test_tensorwise_quant_4096_exact_and_round_trip():
    x = bf16_randn((4096, 4096), seed=209, outlier_frac=0.001)
    q, sinv = turbo.ops.quantize_fp8(x.cuda(), turbo.float8_e4m3, G.TENSORWISE)
    oq, osinv = Q.fp8_tensorwise(x.float().numpy(), "e4m3")
    assert np.array_equal(codes_np(q), oq)
    assert sinv.cpu().view(torch.int32).item() == osinv.view(np.int32).item()
    y = turbo.ops.dequantize_fp8(q, torch.float32, G.TENSORWISE, scale_inv=sinv)
    # within half a step of the e4m3 grid at the value's binade (3 mantissa bits), or of the
    # subnormal step 2^-9, in units of scale_inv
    xf = x.float().cuda()
    step = torch.maximum(torch.abs(xf) * 2.0**-4, sinv * 2.0**-10)
    assert bool(torch.all(torch.abs(y - xf) <= step * 1.0001))


def test_rowwise_quant_8192_sampled_rows_exact():
    x = bf16_randn((8192, 8192), seed=210, scale=0.02)
    q, s = turbo.ops.quantize_fp8(x.cuda(), turbo.float8_e4m3, G.ROWWISE, axis=-1)
    rows = _pick(8192, 512, 9)
    oq, os_ = Q.fp8_rowwise(x.float().numpy()[rows], -1, "e4m3")
    assert np.array_equal(codes_np(q)[rows], oq)
    assert np.array_equal(to_f32_np(s)[rows].view(np.int32), os_.view(np.int32))
    # the other axis, on sampled columns
    qc, sc = turbo.ops.quantize_fp8(x.cuda(), turbo.float8_e4m3, G.ROWWISE, axis=-2)
    cols = _pick(8192, 256, 10)
    oq, os_ = Q.fp8_rowwise(x.float().numpy()[:, cols], 0, "e4m3")
    assert np.array_equal(codes_np(qc)[:, cols], oq)
    assert np.array_equal(to_f32_np(sc)[:, cols].view(np.int32), os_.view(np.int32))


@pytest.mark.parametrize("fp4", [False, True])
def test_mx_quant_16384_sampled_tiles_exact(fp4):
    if fp4 and FP4 is None:
        pytest.skip("torch has no float4_e2m1fn_x2")
    fmt = "e2m1" if fp4 else "e4m3"
    quant = qi.quantize_mxfp4_impl if fp4 else qi.quantize_mxfp8_impl
    qdt = FP4 if fp4 else torch.float8_e4m3fn
    M = N = 16384
    x = bf16_randn((M, N), seed=211, outlier_frac=0.0005)
    xr, sr, xc, sc = quant(x.cuda(), qdt, None, 32, with_trans=True)
    cb = 2 if fp4 else 1  # codes per byte
    for r0 in (0, 4736, M - 128):  # row bands of 128: rows of the row output, columns of the transposed one
        band = x[r0 : r0 + 128].float().numpy()
        oq, os_ = Q.mx_quant_rowwise(band, fmt)
        assert np.array_equal(codes_np(xr)[r0 : r0 + 128], oq)
        assert np.array_equal(codes_np(sr)[r0 : r0 + 128], os_)
        cq, cs = Q.mx_quant_colwise(band, fmt)
        assert np.array_equal(codes_np(xc)[:, r0 // cb : (r0 + 128) // cb], cq[:, : 128 // cb])
        assert np.array_equal(codes_np(sc)[:, r0 // 32 : r0 // 32 + 4], cs[:, :4])
