"""GPU parity of the MoE grouped FP8 GEMM (128-blockwise scales): forward / dgrad product over
row groups, variable-K wgrad product, and the autograd op.

Gate: against the fp32 matmul of the de-quantized operands, max |err| / max |ref| <= 1e-2 and
cosine >= 0.9999 (per call); the op is also held to the reference's SNR gate against the
unquantized bf16 computation (tests/pytorch/ops/test_grouped_gemm_fp8.py of the reference:
25 dB for E4M3 blockwise).
"""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, codes_np, gemm_gate, group_lens, to_f32_np
from oracle import gemm as OG
from oracle import quantize as Q

pytestmark = pytest.mark.gpu

MAX_REL = 1e-2
MIN_COS = 0.9999


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, Float8QuantConfig, Format, gimpl, qimpl
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, Format
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.kernels.grouped_gemm import grouped_gemm_fp8_impl as gimpl
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qimpl


def _gate(ref, got, what=""):
    return gemm_gate(ref, got, what)


def _offs(lens):
    gl = torch.from_numpy(lens).cuda()
    return gl, torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)


CASES = [
    # kind, G, M_total, N, K
    ("balanced", 4, 1024, 512, 384),
    ("ragged", 8, 3000, 384, 512),
    ("zeros", 8, 2048, 256, 1024),
    ("zipf", 32, 8192, 1024, 768),
    ("ragged", 3, 77, 100, 200),  # everything unaligned, K below three slabs
    ("zipf", 16, 4096, 4096, 256),
]


@pytest.mark.parametrize("tile_cfg", [0, 4])
@pytest.mark.parametrize("kind,G_,M,N,K", CASES)
@pytest.mark.parametrize("trans_b", [True, False])
def test_grouped_forward_product(kind, G_, M, N, K, trans_b, tile_cfg):
    """out[rows of g] = A_g . W_g^T from the fused grouped quantizer's row output and 2-D-block
    weights; both weight layouts; empty and ragged groups; automatic tile choice and the pinned
    eight-wavefront 256 x 256 tile."""
    gimpl.TILE_CFG = tile_cfg
    try:
        _grouped_forward_product(kind, G_, M, N, K, trans_b)
    finally:
        gimpl.TILE_CFG = 0


def _grouped_forward_product(kind, G_, M, N, K, trans_b):
    lens = group_lens(kind, G_, M, 31)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=32)
    w = bf16_randn((G_, N, K) if trans_b else (G_, K, N), seed=33)
    qr, _, sr, _, _, _ = qimpl.quant_fp8_blockwise_segment_m_row_col_impl(x.cuda(), torch.float8_e4m3fn, 128, gl, offs, N)
    wq, ws = qimpl.quant_fp8_blockwise_for_weight_impl(w.cuda(), torch.float8_e4m3fn, 128)
    out = gimpl.grouped_gemm_fp8_impl(qr, wq, sr, ws, gl, offs, False, trans_b, torch.bfloat16, G.BLOCKWISE.value, None, 0)
    torch.cuda.synchronize()
    a_deq = Q.fp8_blockwise_dequant(codes_np(qr), np.ascontiguousarray(to_f32_np(sr).T), 1, "e4m3", 128)
    w_deq = np.stack([Q.fp8_blockwise_weight_dequant(codes_np(wq[g]), to_f32_np(ws[g]), "e4m3", 128) for g in range(G_)])
    ref = OG.grouped_gemm_dequantized(a_deq, w_deq, lens, trans_b=trans_b)
    _gate(ref, to_f32_np(out), f"{kind} G={G_} {M}x{N}x{K} trans_b={trans_b}")


def test_grouped_forward_zero_tail_and_determinism():
    """Rows past the last routed token come back zero (the output is allocated for M rows while
    the groups cover fewer); two runs give identical bytes."""
    G_, M, N, K = 4, 1024, 256, 384
    lens = np.array([100, 0, 300, 200], dtype=np.int64)  # 600 of 1024 rows routed
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=34)
    w = bf16_randn((G_, N, K), seed=35)
    qr, _, sr, _, _, _ = qimpl.quant_fp8_blockwise_segment_m_row_col_impl(x.cuda(), torch.float8_e4m3fn, 128, gl, offs, N)
    wq, ws = qimpl.quant_fp8_blockwise_for_weight_impl(w.cuda(), torch.float8_e4m3fn, 128)
    args = (qr, wq, sr, ws, gl, offs, False, True, torch.bfloat16, G.BLOCKWISE.value, None, 0)
    o1 = gimpl.grouped_gemm_fp8_impl(*args)
    o2 = gimpl.grouped_gemm_fp8_impl(*args)
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)
    assert torch.count_nonzero(o1[600:]).item() == 0
    a_deq = Q.fp8_blockwise_dequant(codes_np(qr), np.ascontiguousarray(to_f32_np(sr).T), 1, "e4m3", 128)
    w_deq = np.stack([Q.fp8_blockwise_weight_dequant(codes_np(wq[g]), to_f32_np(ws[g]), "e4m3", 128) for g in range(G_)])
    ref = OG.grouped_gemm_dequantized(a_deq, w_deq, lens, trans_b=True)
    _gate(ref[:600], to_f32_np(o1)[:600], "routed rows")


@pytest.mark.parametrize("kind,G_,M,N,K", CASES[:5])
@pytest.mark.parametrize("trans_c", [True, False])
@pytest.mark.parametrize("tile_cfg", [0, 2, 4])
def test_grouped_variable_k_product(kind, G_, M, N, K, trans_c, tile_cfg):
    """dW[g] = X_g^T . dY_g from the segment-padded column quantizations; an empty group gives
    exactly zero; trans_c returns the transposed product. tile_cfg 4 is the eight-wavefront
    256 x 256 kernel that streams through the groups of a chunk, 2 the 256 x 128 tile: the same
    sums in the same order, so their results are identical."""
    lens = group_lens(kind, G_, M, 36)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=37)
    dy = bf16_randn((M, N), seed=38)
    _, xc, _, xs, plens, poffs = qimpl.quant_fp8_blockwise_segment_m_row_col_impl(x.cuda(), torch.float8_e4m3fn, 128, gl, offs, N)
    _, gc, _, gs, _, _ = qimpl.quant_fp8_blockwise_segment_m_row_col_impl(dy.cuda(), torch.float8_e5m2, 128, gl, offs, K)
    gimpl.TILE_CFG = tile_cfg
    try:
        out = gimpl.grouped_gemm_fp8_variable_k_impl(xc, gc, xs, gs, plens, poffs, True, False, trans_c, torch.bfloat16,
                                                     G.BLOCKWISE.value, None, 0)
        gimpl.TILE_CFG = 3
        out3 = gimpl.grouped_gemm_fp8_variable_k_impl(xc, gc, xs, gs, plens, poffs, True, False, trans_c, torch.bfloat16,
                                                      G.BLOCKWISE.value, None, 0)
    finally:
        gimpl.TILE_CFG = 0
    torch.cuda.synchronize()
    assert torch.equal(out, out3), "tile configurations differ"
    po = poffs.cpu().numpy()
    rows = int(po[-1])
    x_deq = Q.fp8_blockwise_dequant(codes_np(xc)[:rows], to_f32_np(xs)[: rows // 128], 0, "e4m3", 128)
    g_deq = Q.fp8_blockwise_dequant(codes_np(gc)[:rows], to_f32_np(gs)[: rows // 128], 0, "e5m2", 128)
    ref = OG.grouped_gemm_variable_k_dequantized(x_deq, g_deq, np.diff(po))  # pad rows are zero
    if trans_c:
        ref = np.ascontiguousarray(ref.transpose(0, 2, 1))
    got = to_f32_np(out)
    for g in range(G_):
        if lens[g] == 0:
            assert not got[g].any(), f"group {g} is empty: dW must be exactly zero"
    _gate(ref, got, f"{kind} G={G_} trans_c={trans_c}")


@pytest.mark.parametrize("kind,G_,M", [("balanced", 1, 1500), ("zipf", 5, 3000), ("zeros", 64, 6000), ("zipf", 40, 9000)])
@pytest.mark.parametrize("out_dtype,accumulate", [(torch.bfloat16, False), (torch.float32, False), (torch.float32, True)])
def test_grouped_variable_k_streaming_tile_mid_size(kind, G_, M, out_dtype, accumulate):
    """Outputs of 1024 x 1280 (the automatic choice is the eight-wavefront streaming tile; 1280 is
    not a whole number of 256-column tiles, so edge tiles take the checked store path) with one
    group, few groups, more groups than chunks and many empty ones: identical with the 128 x 128
    four-wavefront tile, within the gate of the oracle, empty groups exactly zero / untouched."""
    N, K = 1280, 1024  # dW is [G, N, K] with trans_c
    lens = group_lens(kind, G_, M, 136)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=137)
    dy = bf16_randn((M, N), seed=138)
    _, xc, _, xs, plens, poffs = qimpl.quant_fp8_blockwise_segment_m_row_col_impl(x.cuda(), torch.float8_e4m3fn, 128, gl, offs, N)
    _, gc, _, gs, _, _ = qimpl.quant_fp8_blockwise_segment_m_row_col_impl(dy.cuda(), torch.float8_e5m2, 128, gl, offs, K)

    def run(cfg):
        gimpl.TILE_CFG = cfg
        try:
            if accumulate:
                base = torch.full((G_, N, K), 0.5, dtype=torch.float32, device="cuda")
                gimpl.grouped_gemm_fp8_variable_k_accum_impl(xc, gc, xs, gs, plens, poffs, True, False, True, out_dtype,
                                                             G.BLOCKWISE.value, None, 0, base)
                return base - 0.5
            return gimpl.grouped_gemm_fp8_variable_k_impl(xc, gc, xs, gs, plens, poffs, True, False, True, out_dtype,
                                                          G.BLOCKWISE.value, None, 0)
        finally:
            gimpl.TILE_CFG = 0

    auto, small = run(0), run(3)
    torch.cuda.synchronize()
    if accumulate:  # (x + 0.5) - 0.5 rounds differently from x for small x: compare within fp32 noise
        torch.testing.assert_close(auto, small, rtol=0, atol=1e-5)
    else:
        assert torch.equal(auto, small), "tile configurations differ"
    po = poffs.cpu().numpy()
    rows = int(po[-1])
    x_deq = Q.fp8_blockwise_dequant(codes_np(xc)[:rows], to_f32_np(xs)[: rows // 128], 0, "e4m3", 128)
    g_deq = Q.fp8_blockwise_dequant(codes_np(gc)[:rows], to_f32_np(gs)[: rows // 128], 0, "e5m2", 128)
    ref = np.ascontiguousarray(OG.grouped_gemm_variable_k_dequantized(x_deq, g_deq, np.diff(po)).transpose(0, 2, 1))
    got = to_f32_np(auto)
    for g in range(G_):
        if lens[g] == 0:
            assert not got[g].any(), f"group {g} is empty: its dW must be exactly zero (or untouched)"
    if accumulate:
        assert OG.cosine(ref, got) >= MIN_COS
    else:
        _gate(ref, got, f"{kind} G={G_}")


@pytest.mark.parametrize("tile_cfg", [0, 4])
def test_grouped_variable_k_accumulate(tile_cfg):
    """beta = 1: the product is added to an fp32 buffer; empty groups leave theirs unchanged."""
    G_, M, N, K = 4, 1024, 256, 384
    lens = np.array([256, 0, 500, 268], dtype=np.int64)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=39)
    dy = bf16_randn((M, N), seed=40)
    _, xc, _, xs, plens, poffs = qimpl.quant_fp8_blockwise_segment_m_row_col_impl(x.cuda(), torch.float8_e4m3fn, 128, gl, offs, N)
    _, gc, _, gs, _, _ = qimpl.quant_fp8_blockwise_segment_m_row_col_impl(dy.cuda(), torch.float8_e4m3fn, 128, gl, offs, K)
    base = torch.randn((G_, N, K), generator=torch.Generator().manual_seed(41)).cuda()
    acc = base.clone()
    gimpl.TILE_CFG = tile_cfg
    try:
        fresh = gimpl.grouped_gemm_fp8_variable_k_impl(xc, gc, xs, gs, plens, poffs, True, False, True, torch.float32,
                                                       G.BLOCKWISE.value, None, 0)
        gimpl.grouped_gemm_fp8_variable_k_accum_impl(xc, gc, xs, gs, plens, poffs, True, False, True, torch.float32,
                                                     G.BLOCKWISE.value, None, 0, acc)
    finally:
        gimpl.TILE_CFG = 0
    torch.cuda.synchronize()
    assert torch.equal(acc[1], base[1])
    torch.testing.assert_close(acc, base + fresh, rtol=1e-6, atol=1e-5)


@pytest.mark.parametrize("trans_b", [True, False])
def test_grouped_gemm_fp8_autograd(trans_b):
    """The op end to end (quantize, forward, dgrad, wgrad) against the bf16 grouped matmul: the
    reference's 25 dB SNR gate for E4M3 blockwise; empty experts get a zero weight gradient."""
    G_, M, N, K = 8, 4096, 1024, 512
    lens = group_lens("zipf", G_, M, 42)
    gl, _ = _offs(lens)
    a = bf16_randn((M, K), seed=43).cuda().requires_grad_(True)
    b = bf16_randn((G_, N, K) if trans_b else (G_, K, N), seed=44).cuda().requires_grad_(True)
    cfg = Float8QuantConfig(format=Format.E4M3, granularity=G.BLOCKWISE, block_size=128)
    out = turbo.ops.grouped_gemm_fp8(a, b, gl, trans_b=trans_b, config=cfg)
    dy = bf16_randn((M, N), seed=45).cuda()
    out.backward(dy)
    torch.cuda.synchronize()

    af, bf_, dyf = to_f32_np(a), to_f32_np(b), to_f32_np(dy)
    ref_out = OG.grouped_gemm_dequantized(af, bf_, lens, trans_b=trans_b)
    ref_da = OG.grouped_gemm_dequantized(dyf, bf_, lens, trans_b=not trans_b)
    ref_db = OG.grouped_gemm_variable_k_dequantized(af, dyf, lens)  # [G, K, N]
    if trans_b:
        ref_db = ref_db.transpose(0, 2, 1)
    assert OG.snr_db(ref_out, to_f32_np(out)) > 25
    assert OG.snr_db(ref_da, to_f32_np(a.grad)) > 25
    assert OG.snr_db(ref_db, to_f32_np(b.grad)) > 25
    for g in range(G_):
        if lens[g] == 0:
            assert torch.count_nonzero(b.grad[g]).item() == 0


@pytest.mark.parametrize("kind,G_,M,N,K", CASES[:5])
@pytest.mark.parametrize("trans_c", [True, False])
def test_grouped_variable_k_kmajor_operands(kind, G_, M, N, K, trans_c):
    """The variable-K product over operands that arrive transposed (``trans_a=False, trans_b=True``:
    the transposed column output of the grouped quantizer) is bit-identical to the product that
    transposes the untransposed ones itself, also with the beta = 1 epilogue."""
    lens = group_lens(kind, G_, M, 39)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=40).cuda()
    dy = bf16_randn((M, N), seed=41).cuda()
    seg, seg_t = qimpl.quant_fp8_blockwise_segment_m_row_col_impl, qimpl.quant_fp8_blockwise_segment_m_row_col_t_impl
    _, xc, _, xs, plens, poffs = seg(x, torch.float8_e4m3fn, 128, gl, offs, N)
    _, gc, _, gs, _, _ = seg(dy, torch.float8_e5m2, 128, gl, offs, K)
    _, xct, _, xs2, _, _ = seg_t(x, torch.float8_e4m3fn, 128, gl, offs)
    _, gct, _, gs2, _, _ = seg_t(dy, torch.float8_e5m2, 128, gl, offs)
    args = (plens, poffs)
    ref = gimpl.grouped_gemm_fp8_variable_k_impl(xc, gc, xs, gs, *args, True, False, trans_c, torch.bfloat16,
                                                 G.BLOCKWISE.value, None, 0)
    out = gimpl.grouped_gemm_fp8_variable_k_impl(xct, gct, xs2, gs2, *args, False, True, trans_c, torch.bfloat16,
                                                 G.BLOCKWISE.value, None, 0)
    torch.cuda.synchronize()
    assert out.shape == ref.shape and torch.equal(out, ref)
    acc = torch.full(ref.shape, 0.5, dtype=torch.float32, device="cuda")
    acc_ref = acc.clone()
    gimpl.grouped_gemm_fp8_variable_k_accum_impl(xct, gct, xs2, gs2, *args, False, True, trans_c, torch.float32,
                                                 G.BLOCKWISE.value, None, 0, acc)
    gimpl.grouped_gemm_fp8_variable_k_accum_impl(xc, gc, xs, gs, *args, True, False, trans_c, torch.float32,
                                                 G.BLOCKWISE.value, None, 0, acc_ref)
    assert torch.equal(acc, acc_ref)
