"""GPU parity of the grouped FP8 GEMM with vector scales (TENSORWISE / ROWWISE): forward / dgrad
products over row groups (both weight layouts) and the variable-K wgrad over tightly packed groups
against the fp32 matmul of the de-quantized operands (max |err| / max |ref| <= 1e-2, cosine >=
0.9999), and the autograd op at the reference's SNR gates against the unquantized computation
(tests/pytorch/ops/test_grouped_gemm_fp8.py of the reference: 25 dB E4M3, 20 dB E5M2 / HYBRID)."""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, codes_np, gemm_gate, group_lens, to_f32_np
from oracle import gemm as OG
from oracle import quantize as Q

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, Float8QuantConfig, Format, gimpl
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, Format
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.kernels.grouped_gemm import grouped_gemm_fp8_impl as gimpl


def _gate(ref, got, what=""):
    return gemm_gate(ref, got, what)


def _offs(lens):
    gl = torch.from_numpy(lens).cuda()
    return gl, torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)


def _deq(q, s):
    return Q.fp8_dequant(codes_np(q), to_f32_np(s), "e4m3")


CASES = [("balanced", 4, 1024, 512, 384), ("ragged", 8, 3000, 384, 512), ("zeros", 8, 2048, 256, 1024),
         ("zipf", 32, 8192, 1024, 768), ("ragged", 3, 77, 100, 200), ("zipf", 16, 4096, 2048, 256)]


@pytest.mark.parametrize("kind,G_,M,N,K", CASES)
@pytest.mark.parametrize("gran", ["ROWWISE", "TENSORWISE"])
@pytest.mark.parametrize("trans_b", [True, False])
def test_grouped_vec_forward_product(kind, G_, M, N, K, gran, trans_b):
    gr = getattr(G, gran)
    lens = group_lens(kind, G_, M, 61)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=62).cuda()
    w = bf16_randn((G_, N, K) if trans_b else (G_, K, N), seed=63).cuda()
    xq, xs = turbo.ops.quantize_fp8(x, turbo.float8_e4m3, gr, axis=-1)
    wq, ws = turbo.ops.quantize_fp8(w, turbo.float8_e4m3, gr, axis=-1 if trans_b else -2)
    out = gimpl.grouped_gemm_fp8_impl(xq, wq, xs, ws, gl, offs, False, trans_b, torch.bfloat16, gr.value, None, 0)
    torch.cuda.synchronize()
    ref = OG.grouped_gemm_dequantized(_deq(xq, xs), _deq(wq, ws), lens, trans_b=trans_b)
    _gate(ref, to_f32_np(out), f"{gran} {kind} G={G_} {M}x{N}x{K} trans_b={trans_b}")


@pytest.mark.parametrize("kind,G_,M,N,K", CASES)
@pytest.mark.parametrize("gran", ["ROWWISE", "TENSORWISE"])
@pytest.mark.parametrize("trans_c", [False, True])
def test_grouped_vec_variable_k_product(kind, G_, M, N, K, gran, trans_c):
    gr = getattr(G, gran)
    lens = group_lens(kind, G_, M, 64)
    gl, offs = _offs(lens)
    x = bf16_randn((M, K), seed=65).cuda()
    dy = bf16_randn((M, N), seed=66).cuda()
    xq, xs = turbo.ops.quantize_fp8(x, turbo.float8_e4m3, gr, axis=-2)
    gq, gs = turbo.ops.quantize_fp8(dy, turbo.float8_e5m2, gr, axis=-2)
    out = gimpl.grouped_gemm_fp8_variable_k_impl(xq, gq, xs, gs, gl, offs, True, False, trans_c, torch.float32, gr.value,
                                                 None, 0)
    torch.cuda.synchronize()
    ref = OG.grouped_gemm_variable_k_dequantized(_deq(xq, xs), Q.fp8_dequant(codes_np(gq), to_f32_np(gs), "e5m2"), lens)
    if trans_c:
        ref = np.ascontiguousarray(ref.transpose(0, 2, 1))
    _gate(ref, to_f32_np(out), f"{gran} variable-K {kind} G={G_}")
    for g in range(G_):
        if lens[g] == 0:
            assert not bool(out[g].abs().max() > 0)
    acc = torch.ones_like(out)
    gimpl.grouped_gemm_fp8_variable_k_accum_impl(xq, gq, xs, gs, gl, offs, True, False, trans_c, torch.float32, gr.value,
                                                 None, 0, acc)
    assert torch.allclose(acc, out + 1, rtol=0, atol=1e-3 * float(out.abs().max()) + 1e-6)


@pytest.mark.parametrize("gran", ["ROWWISE", "TENSORWISE"])
@pytest.mark.parametrize("fmt,gate", [("E4M3", 25), ("E5M2", 20), ("HYBRID", 20)])
@pytest.mark.parametrize("trans_b", [True, False])
def test_grouped_gemm_fp8_vec_autograd(gran, fmt, gate, trans_b):
    G_, M, N, K = 8, 4096, 1024, 512
    lens = group_lens("zipf", G_, M, 67)
    gl, _ = _offs(lens)
    a = bf16_randn((M, K), seed=68).cuda().requires_grad_(True)
    b = bf16_randn((G_, N, K) if trans_b else (G_, K, N), seed=69).cuda().requires_grad_(True)
    cfg = Float8QuantConfig(format=getattr(Format, fmt), granularity=getattr(G, gran))
    out = turbo.ops.grouped_gemm_fp8(a, b, gl, trans_b=trans_b, config=cfg)
    dy = bf16_randn((M, N), seed=70).cuda()
    out.backward(dy)
    torch.cuda.synchronize()
    af, bf_, dyf = to_f32_np(a), to_f32_np(b), to_f32_np(dy)
    ref_out = OG.grouped_gemm_dequantized(af, bf_, lens, trans_b=trans_b)
    ref_da = OG.grouped_gemm_dequantized(dyf, bf_, lens, trans_b=not trans_b)
    ref_db = OG.grouped_gemm_variable_k_dequantized(af, dyf, lens)  # [G, K, N]
    if trans_b:
        ref_db = ref_db.transpose(0, 2, 1)
    assert OG.snr_db(ref_out, to_f32_np(out)) > gate
    assert OG.snr_db(ref_da, to_f32_np(a.grad)) > gate
    assert OG.snr_db(ref_db, to_f32_np(b.grad)) > gate
    for g in range(G_):
        if lens[g] == 0:
            assert torch.count_nonzero(b.grad[g]).item() == 0


@pytest.mark.parametrize("gran", ["TENSORWISE", "ROWWISE", "BLOCKWISE", "MX_BLOCKWISE"])
@pytest.mark.parametrize("main_dtype", [torch.float32, torch.bfloat16])
def test_grouped_gemm_fp8_fused_grad_accum(gran, main_dtype):
    """``fuse_bgrad_accum_pattern="megatron"`` for every grouped FP8 granularity: the wgrad GEMM adds
    into ``b.main_grad`` (beta = 1 epilogue), flags the weight, and autograd receives a placeholder;
    ``main_grad`` ends as previous + the gradient of the unfused call
    (reference: primus_turbo/pytorch/ops/utils.py:37-89 and its callers in ops/grouped_gemm_fp8.py)."""
    from primus_turbo.pytorch.core.low_precision import ScaleDtype

    g = getattr(G, gran)
    kw = {"BLOCKWISE": dict(block_size=128), "MX_BLOCKWISE": dict(block_size=32, scale_dtype=ScaleDtype.E8M0)}.get(gran, {})
    cfg = Float8QuantConfig(format=Format.E4M3, granularity=g, **kw)
    lens = group_lens("ragged", 4, 1024, 91)
    gl, _ = _offs(lens)
    a = bf16_randn((1024, 512), seed=92).cuda().requires_grad_(True)
    b = bf16_randn((4, 768, 512), seed=93).cuda().requires_grad_(True)
    dy = bf16_randn((1024, 768), seed=94).cuda()
    turbo.ops.grouped_gemm_fp8(a, b, gl, trans_b=True, config=cfg).backward(dy)
    plain, plain_da = b.grad.clone(), a.grad.clone()
    a.grad = b.grad = None
    b.main_grad = torch.full((4, 768, 512), 0.25, dtype=main_dtype, device="cuda")
    b.grad_added_to_main_grad = False
    turbo.ops.grouped_gemm_fp8(a, b, gl, trans_b=True, config=cfg, fuse_bgrad_accum_pattern="megatron").backward(dy)
    torch.cuda.synchronize()
    assert b.grad_added_to_main_grad and torch.equal(a.grad, plain_da)
    want = plain.float() + 0.25
    # fp32 accumulators differ from the unfused bf16 result by its rounding; bf16 ones round once more
    tol = (2.0 ** -7 if main_dtype == torch.bfloat16 else 2.0 ** -8) * float(want.abs().max())
    assert torch.allclose(b.main_grad.float(), want, rtol=0, atol=tol)
    with pytest.raises(AssertionError):
        c = bf16_randn((4, 768, 512), seed=95).cuda().requires_grad_(True)  # no main_grad set up
        turbo.ops.grouped_gemm_fp8(a, c, gl, trans_b=True, config=cfg, fuse_bgrad_accum_pattern="megatron")
