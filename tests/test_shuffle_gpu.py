"""GPU parity of the pre-shuffled MX layouts against oracle/shuffle.py, bit-exact (bytes only).
Follows the reference's tests/pytorch/ops/test_quantization.py:486-548 (MXFP8, scales) and :688-762
(MXFP4, codes and scales): the quantizers' ``shuffle_scale`` / ``shuffle_out`` outputs equal the
stand-alone ``shuffle_scale`` / ``shuffle_weight`` ops applied to the plain outputs, for B x M x N in
{1, 4} x {32 ... 1024}^2 viewed as 2-D, with and without 2-D blocks. Added here: both against the
oracle, the inverse passes, ragged scale shapes, and GEMMs on pre-shuffled operands."""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, codes_np
from oracle import shuffle as S

pytestmark = pytest.mark.gpu

FP4 = getattr(torch, "float4_e2m1fn_x2", None)
E8M0 = getattr(torch, "float8_e8m0fnu", None)
needs_fp4 = pytest.mark.skipif(FP4 is None or E8M0 is None, reason="torch has no float4_e2m1fn_x2 / float8_e8m0fnu")


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, ext, ScalingRecipe, G, qi
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G, ScalingRecipe
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

    ext = torch.ops.primus_turbo_cpp_extension


def _bytes(shape, seed):
    return torch.from_numpy(np.random.default_rng(seed).integers(0, 256, shape, dtype=np.uint8))


@needs_fp4
@pytest.mark.parametrize("M,N", [(32, 8), (256, 8), (100, 5), (300, 12), (1, 1), (1024, 32), (4096, 224)])
def test_shuffle_scale_op_matches_oracle(M, N):
    s = _bytes((M, N), M * 131 + N)
    got = ext.shuffle_scale(s.cuda().view(E8M0), [16, 16])
    want = S.shuffle_scale(s.numpy())
    assert got.dtype == E8M0 and tuple(got.shape) == want.shape
    assert np.array_equal(codes_np(got), want)
    back = ext.unshuffle_scale(got, M, N)
    assert np.array_equal(codes_np(back), s.numpy())


@needs_fp4
@pytest.mark.parametrize("M,N", [(16, 32), (32, 64), (48, 160), (1024, 512), (4096, 4096)])
def test_shuffle_weight_op_matches_oracle(M, N):
    w = _bytes((M, N), M * 7 + N)
    got = ext.shuffle_weight(w.cuda().view(FP4), [16, 16])
    assert got.dtype == FP4 and tuple(got.shape) == (M, N)
    assert np.array_equal(codes_np(got), S.shuffle_codes(w.numpy()))
    assert np.array_equal(codes_np(ext.unshuffle_weight(got, [16, 16])), w.numpy())


@needs_fp4
def test_shuffle_op_argument_checks():
    w = _bytes((24, 64), 1).cuda().view(FP4)
    with pytest.raises(RuntimeError, match="M must be divisible by 16"):
        ext.shuffle_weight(w, [16, 16])
    with pytest.raises(RuntimeError, match="N must be divisible by 32"):
        ext.shuffle_weight(_bytes((32, 48), 2).cuda().view(FP4), [16, 16])
    with pytest.raises(RuntimeError, match="Unsupported shuffle layout"):
        ext.shuffle_weight(_bytes((32, 64), 3).cuda().view(FP4), [32, 16])
    with pytest.raises(RuntimeError, match="Float8_e8m0fnu"):
        ext.shuffle_scale(_bytes((32, 8), 4).cuda(), [16, 16])
    with pytest.raises(RuntimeError, match="exactly 2 elements"):
        ext.shuffle_scale(_bytes((32, 8), 4).cuda().view(E8M0), [16])


def _expect(q, s, shuffle_out, shuffle_scale):
    """Oracle layouts of one direction's plain outputs (2-D)."""
    qn, sn = codes_np(q), codes_np(s)
    return (S.shuffle_codes(qn) if shuffle_out else qn), (S.shuffle_scale(sn) if shuffle_scale else sn)


@needs_fp4
@pytest.mark.parametrize("B,M,N", [(1, 32, 32), (1, 64, 1024), (4, 256, 64), (4, 1024, 256), (1, 1024, 1024)])
@pytest.mark.parametrize("use_2d_block", [True, False])
def test_quantize_mxfp4_shuffle(B, M, N, use_2d_block):
    x = bf16_randn((B * M, N), seed=42 + M + N).cuda()
    plain = ScalingRecipe(use_2d_block=use_2d_block)
    shuf = ScalingRecipe(use_2d_block=use_2d_block, shuffle_scale=True, shuffle_out=True)
    kw = dict(granularity=G.MX_BLOCKWISE, block_size=32)
    rq, rs, cq, cs = turbo.ops.quantize_fp4_with_trans(x, FP4, scaling_recipe=plain, scaling_recipe_for_trans=plain, **kw)
    srq, srs, scq, scs = turbo.ops.quantize_fp4_with_trans(x, FP4, scaling_recipe=shuf, scaling_recipe_for_trans=shuf, **kw)
    for got_q, got_s, q, s, what in ((srq, srs, rq, rs, "rowwise"), (scq, scs, cq, cs, "colwise")):
        want_q, want_s = _expect(q, s, True, True)
        assert np.array_equal(codes_np(got_q), want_q), f"{what} codes"
        assert np.array_equal(codes_np(got_s), want_s), f"{what} scales"
        # the reference's own check: fused outputs == stand-alone ops on the plain outputs
        assert torch.equal(got_q.view(torch.uint8), ext.shuffle_weight(q, [16, 16]).view(torch.uint8))
        assert torch.equal(got_s.view(torch.uint8), ext.shuffle_scale(s, [16, 16]).view(torch.uint8))
    # one direction, scales only (the layout of the first operand of a pre-shuffled product)
    q1, s1 = turbo.ops.quantize_fp4(x, FP4, axis=1, **kw,
                                    scaling_recipe=ScalingRecipe(use_2d_block=use_2d_block, shuffle_scale=True))
    want_q, want_s = _expect(rq, rs, False, True)
    assert np.array_equal(codes_np(q1), want_q) and np.array_equal(codes_np(s1), want_s)


@needs_fp4
@pytest.mark.parametrize("B,M,N", [(1, 32, 32), (4, 256, 64), (1, 1024, 1024)])
@pytest.mark.parametrize("dt", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_quantize_mxfp8_shuffle(B, M, N, dt):
    x = bf16_randn((B * M, N), seed=7 + M + N).cuda()
    kw = dict(granularity=G.MX_BLOCKWISE, block_size=32)
    plain, shuf = ScalingRecipe(), ScalingRecipe(shuffle_scale=True)
    rq, rs, cq, cs = turbo.ops.quantize_fp8_with_trans(x, dt, scaling_recipe=plain, scaling_recipe_for_trans=plain, **kw)
    srq, srs, scq, scs = turbo.ops.quantize_fp8_with_trans(x, dt, scaling_recipe=shuf, scaling_recipe_for_trans=shuf, **kw)
    assert torch.equal(srq.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(scq.view(torch.uint8), cq.view(torch.uint8))
    assert np.array_equal(codes_np(srs), S.shuffle_scale(codes_np(rs)))
    assert np.array_equal(codes_np(scs), S.shuffle_scale(codes_np(cs)))
    both = ScalingRecipe(shuffle_scale=True, shuffle_out=True)
    bq, bs_ = turbo.ops.quantize_fp8(x, dt, axis=1, scaling_recipe=both, **kw)
    assert np.array_equal(codes_np(bq), S.shuffle_codes(codes_np(rq))) and np.array_equal(codes_np(bs_), codes_np(srs))


@needs_fp4
def test_quantize_mxfp4_shuffle_batched_scales_pad_per_matrix():
    B, M, N = 3, 48, 64
    x = bf16_randn((B, M, N), seed=9).cuda()
    q, s = qi.quantize_mxfp4_impl(x, FP4, 2, 32, scaling_recipe=ScalingRecipe(shuffle_scale=True, shuffle_out=True))
    pq, ps = qi.quantize_mxfp4_impl(x, FP4, 2, 32, scaling_recipe=ScalingRecipe())
    assert tuple(s.shape) == (B, 256, 8) and tuple(q.shape) == tuple(pq.shape)
    for b in range(B):
        assert np.array_equal(codes_np(s[b]), S.shuffle_scale(codes_np(ps[b])))
    # 48 rows per matrix = whole bands of 16, so the flattened rows shuffle band by band
    assert np.array_equal(codes_np(q).reshape(B * M, -1), S.shuffle_codes(codes_np(pq).reshape(B * M, -1)))


@needs_fp4
def test_dequantize_shuffled_round_trip():
    x = bf16_randn((256, 512), seed=11).cuda()
    kw = dict(granularity=G.MX_BLOCKWISE, block_size=32)
    shuf = ScalingRecipe(shuffle_scale=True, shuffle_out=True)
    q, s = turbo.ops.quantize_fp4(x, FP4, axis=1, scaling_recipe=shuf, **kw)
    pq, ps = turbo.ops.quantize_fp4(x, FP4, axis=1, scaling_recipe=ScalingRecipe(), **kw)
    d = turbo.ops.dequantize_fp4(q, torch.bfloat16, axis=1, scale_inv=s, scaling_recipe=shuf, **kw)
    dp = turbo.ops.dequantize_fp4(pq, torch.bfloat16, axis=1, scale_inv=ps, scaling_recipe=ScalingRecipe(), **kw)
    assert torch.equal(d, dp)


@needs_fp4
def test_gemm_fp4_preshuffled_operands_give_the_plain_result():
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig
    from primus_turbo.pytorch.core.quantized_tensor import QuantizedTensor, QuantizedTensorPair
    from primus_turbo.pytorch.kernels.gemm.gemm_fp4_impl import gemm_fp4_impl

    M, Nn, K = 256, 384, 512
    a = bf16_randn((M, K), seed=21).cuda()
    b = bf16_randn((Nn, K), seed=22).cuda()
    kw = dict(granularity=G.MX_BLOCKWISE, block_size=32)
    aq, as_ = turbo.ops.quantize_fp4(a, FP4, axis=1, scaling_recipe=ScalingRecipe(), **kw)
    bq, bs_ = turbo.ops.quantize_fp4(b, FP4, axis=1, scaling_recipe=ScalingRecipe(use_2d_block=True), **kw)
    ref = gemm_fp4_impl(aq, as_, False, bq, bs_, True, torch.bfloat16, False, G.MX_BLOCKWISE.value, 0)
    # impl level: a = plain codes + shuffled scales, b = shuffled codes and scales (the reference's AITER call)
    saq, sas = turbo.ops.quantize_fp4(a, FP4, axis=1, scaling_recipe=ScalingRecipe(shuffle_scale=True), **kw)
    sbq, sbs = turbo.ops.quantize_fp4(b, FP4, axis=1, scaling_recipe=ScalingRecipe(use_2d_block=True, shuffle_scale=True,
                                                                                 shuffle_out=True), **kw)
    out = gemm_fp4_impl(saq, sas, False, sbq, sbs, True, torch.bfloat16, False, G.MX_BLOCKWISE.value, 0, preshuffled=True)
    assert torch.equal(out, ref)

    # op level: use_preshuffle changes no result, with plain tensors ...
    plain_cfg, pre_cfg = Float4QuantConfig(), Float4QuantConfig(use_preshuffle=True)

    def run(cfg, a_in, b_in):
        a_leaf = a.clone().requires_grad_(True)
        b_leaf = b.clone().requires_grad_(True)
        y = turbo.ops.gemm_fp4(a_leaf if a_in is None else a_in, b_leaf if b_in is None else b_in, False, True,
                               torch.bfloat16, cfg)
        y.float().sum().backward()
        return y.detach(), a_leaf.grad, b_leaf.grad

    y0, ga0, gb0 = run(plain_cfg, None, None)
    y1, ga1, gb1 = run(pre_cfg, None, None)
    assert torch.equal(y0, y1) and torch.equal(ga0, ga1) and torch.equal(gb0, gb1)
    assert torch.equal(y0, ref)
    # ... and with a weight quantized ahead of time in the pre-shuffled layout
    w_recipe = ScalingRecipe(use_2d_block=True, shuffle_scale=True, shuffle_out=True)
    wq = QuantizedTensor.quantize(b, FP4, G.MX_BLOCKWISE, axis=-1, block_size=32, scaling_recipe=w_recipe)
    wq_t = QuantizedTensor.quantize(b, FP4, G.MX_BLOCKWISE, axis=-2, block_size=32, scaling_recipe=w_recipe)
    y2, ga2, _ = run(pre_cfg, None, QuantizedTensorPair(wq, wq_t))
    assert torch.equal(y2, y0) and torch.equal(ga2, ga0)
    assert torch.equal(wq.dequantize(), QuantizedTensor.quantize(
        b, FP4, G.MX_BLOCKWISE, axis=-1, block_size=32, scaling_recipe=ScalingRecipe(use_2d_block=True)).dequantize())
