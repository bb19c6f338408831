"""GPU parity of the MX quantizers (MXFP8 E4M3 / E5M2, MXFP4 E2M1): codes and E8M0 scale
bytes bit-exact against the oracle, single direction and dual, 1-D (1 x 32) and 2-D (32 x 32)
blocks, padded and batched shapes, special values; de-quantizers bit-exact as well."""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, codes_np, to_f32_np
from oracle import quantize as Q

pytestmark = pytest.mark.gpu

FP4 = getattr(torch, "float4_e2m1fn_x2", None)
FMTS = [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)] + ([("e2m1", FP4)] if FP4 is not None else [])


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global qi, ScalingRecipe, turbo, G
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.core.low_precision import ScalingRecipe
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi


def _fn(fmt):
    return qi.quantize_mxfp4_impl if fmt == "e2m1" else qi.quantize_mxfp8_impl


def _dq(fmt):
    return qi.dequantize_mxfp4_impl if fmt == "e2m1" else qi.dequantize_mxfp8_impl


SHAPES = [(128, 128), (256, 512), (200, 96), (33, 32), (1000, 2080), (4096, 1024)]


@pytest.mark.parametrize("fmt,dt", FMTS)
@pytest.mark.parametrize("two_d", [False, True])
@pytest.mark.parametrize("M,N", SHAPES)
def test_mx_dual_matches_oracle(fmt, dt, two_d, M, N):
    x = bf16_randn((M, N), seed=50, outlier_frac=0.002)
    rec = ScalingRecipe(use_2d_block=two_d)
    rq, rs, cq, cs = _fn(fmt)(x.cuda(), dt, None, 32, with_trans=True, scaling_recipe=rec, scaling_recipe_for_trans=rec)
    torch.cuda.synchronize()
    xf = to_f32_np(x)
    oq, os_ = Q.mx_quant_rowwise(xf, fmt, two_d)
    assert codes_np(rq).shape == oq.shape and codes_np(rs).shape == os_.shape
    assert np.array_equal(codes_np(rs), os_), "row scale bytes"
    assert np.array_equal(codes_np(rq), oq), "row codes"
    oq, os_ = Q.mx_quant_colwise(xf, fmt, two_d)
    assert codes_np(cq).shape == oq.shape and codes_np(cs).shape == os_.shape
    assert np.array_equal(codes_np(cs), os_), "col scale bytes"
    assert np.array_equal(codes_np(cq), oq), "col codes"


@pytest.mark.parametrize("fmt,dt", FMTS)
@pytest.mark.parametrize("axis", [0, 1])
def test_mx_single_direction_and_mixed_recipes(fmt, dt, axis):
    """One direction equals the matching half of the dual call; the two directions of a dual
    call may use different block shapes (1-D activations rows, 2-D columns)."""
    x = bf16_randn((384, 256), seed=51).cuda()
    q, s = _fn(fmt)(x, dt, axis, 32)
    rq, rs, cq, cs = _fn(fmt)(x, dt, None, 32, with_trans=True)
    want_q, want_s = (rq, rs) if axis == 1 else (cq, cs)
    assert torch.equal(q.view(torch.uint8), want_q.view(torch.uint8)) and torch.equal(s.view(torch.uint8), want_s.view(torch.uint8))
    rq, rs, cq, cs = _fn(fmt)(x, dt, None, 32, with_trans=True, scaling_recipe=ScalingRecipe(),
                              scaling_recipe_for_trans=ScalingRecipe(use_2d_block=True))
    xf = to_f32_np(x)
    oq, os_ = Q.mx_quant_rowwise(xf, fmt, False)
    assert np.array_equal(codes_np(rq), oq) and np.array_equal(codes_np(rs), os_)
    oq, os_ = Q.mx_quant_colwise(xf, fmt, True)
    assert np.array_equal(codes_np(cq), oq) and np.array_equal(codes_np(cs), os_)


@pytest.mark.parametrize("fmt,dt", FMTS)
@pytest.mark.parametrize("shape,dtype", [((128, 128), torch.bfloat16), ((200, 96), torch.bfloat16),
                                         ((33, 32), torch.float16), ((1000, 2080), torch.bfloat16),
                                         ((7, 4096), torch.bfloat16), ((3, 160, 192), torch.float16),
                                         ((2, 50, 544), torch.bfloat16)])
def test_mx_row_direction_alone(fmt, dt, shape, dtype):
    """Rows only with 1-D blocks (the streaming kernel): codes, the zero codes of the pad columns
    and the scale bytes bit-exact against the oracle, batches and rows shorter than a
    wavefront's share included."""
    x = bf16_randn(shape, seed=58, outlier_frac=0.002, dtype=dtype)
    q, s = _fn(fmt)(x.cuda(), dt, x.ndim - 1, 32)
    torch.cuda.synchronize()
    xs = x if x.ndim == 3 else x[None]
    qs, ss = (q, s) if x.ndim == 3 else (q[None], s[None])
    for b in range(xs.shape[0]):
        oq, os_ = Q.mx_quant_rowwise(to_f32_np(xs[b]), fmt)
        assert codes_np(qs[b]).shape == oq.shape and codes_np(ss[b]).shape == os_.shape
        assert np.array_equal(codes_np(ss[b]), os_), "row scale bytes"
        assert np.array_equal(codes_np(qs[b]), oq), "row codes"


@pytest.mark.parametrize("fmt,dt", FMTS)
def test_mx_row_direction_alone_random_shapes(fmt, dt):
    """Forty random shapes (rows 1 .. 700, columns a multiple of 32 up to 4800, a few batched):
    the row direction quantized alone gives the bytes of the dual quantizer's row output."""
    rng = np.random.default_rng(60)
    for k in range(40):
        M, N = int(rng.integers(1, 701)), 32 * int(rng.integers(1, 151))
        shape = (int(rng.integers(2, 4)), M, N) if k % 8 == 7 else (M, N)
        x = bf16_randn(shape, seed=600 + k, outlier_frac=0.001, dtype=torch.float16 if k % 5 == 4 else torch.bfloat16).cuda()
        q, s = _fn(fmt)(x, dt, x.ndim - 1, 32)
        rq, rs, _, _ = _fn(fmt)(x, dt, None, 32, with_trans=True)
        assert torch.equal(q.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(s.view(torch.uint8), rs.view(torch.uint8)), shape


@pytest.mark.skipif(FP4 is None, reason="torch has no float4_e2m1fn_x2")
@pytest.mark.parametrize("shape", [(256, 128), (3, 200, 608)])
def test_mxfp4_stochastic_rounding_same_noise_alone_and_dual(shape):
    """With one seed the row direction draws the same rounding noise whether it is quantized
    alone (streaming kernel) or together with the column direction (tile kernel)."""
    from primus_turbo import _native as N

    x = bf16_randn(shape, seed=59).cuda()
    B = shape[0] if len(shape) == 3 else 1
    M, Nn = shape[-2:]
    Mp, Np = -(-M // 128) * 128, -(-Nn // 128) * 128
    outs = []
    for dual in (False, True):
        rq = torch.zeros((B, M, Np // 2), dtype=torch.uint8, device="cuda")
        rs = torch.zeros((B, M, Np // 32), dtype=torch.uint8, device="cuda")
        cq = torch.zeros((B, Nn, Mp // 2), dtype=torch.uint8, device="cuda") if dual else None
        cs = torch.zeros((B, Nn, Mp // 32), dtype=torch.uint8, device="cuda") if dual else None
        N.check(N.lib().pt_quantize_mx(N.ptr(x), N.dtype_code(x.dtype), B, M, Nn, N.dtype_code(FP4), N.ptr(rq), N.ptr(rs), 4,
                                       N.ptr(cq), N.ptr(cs), 0, 0x1234ABCD, N.stream_of(x)))
        torch.cuda.synchronize()
        outs.append((rq, rs))
    assert torch.equal(outs[0][1], outs[1][1]) and torch.equal(outs[0][0], outs[1][0])
    q0, _ = qi.quantize_mxfp4_impl(x, FP4, x.ndim - 1, 32)
    assert not torch.equal(outs[0][0], q0.view(torch.uint8).reshape(outs[0][0].shape)), "the noise is there"


@pytest.mark.parametrize("fmt,dt", FMTS)
def test_mx_batched_and_fp16(fmt, dt):
    x = bf16_randn((3, 160, 192), seed=52, dtype=torch.float16)
    rq, rs, cq, cs = _fn(fmt)(x.cuda(), dt, None, 32, with_trans=True)
    assert rq.shape[0] == 3 and cq.shape[0] == 3
    for b in range(3):
        xf = to_f32_np(x[b])
        oq, os_ = Q.mx_quant_rowwise(xf, fmt)
        assert np.array_equal(codes_np(rq[b]), oq) and np.array_equal(codes_np(rs[b]), os_)
        oq, os_ = Q.mx_quant_colwise(xf, fmt)
        assert np.array_equal(codes_np(cq[b]), oq) and np.array_equal(codes_np(cs[b]), os_)


@pytest.mark.parametrize("fmt,dt", FMTS)
def test_mx_special_values(fmt, dt):
    """All-zero blocks (scale byte 0), huge and tiny magnitudes, NaN and inf elements, exact
    ties between representable codes."""
    x = torch.zeros((128, 256), dtype=torch.float32)
    x[0, :32] = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0, 6.0] * 4)  # FP4 midpoints at scale 1
    x[1, :32] = torch.linspace(-7, 7, 32)
    x[2, 32:64] = 3.0e38
    x[3, 64:96] = 1.0e-38
    x[4, 5] = float("nan")
    x[4, 6] = 2.0
    x[5, 40] = float("inf")
    x[5, 41] = -1.0
    x[6, :] = torch.randn(256, generator=torch.Generator().manual_seed(53)) * 1e4
    x[7, 96:128] = -0.0
    xb = x.to(torch.bfloat16)
    rq, rs, cq, cs = _fn(fmt)(xb.cuda(), dt, None, 32, with_trans=True)
    xf = to_f32_np(xb)
    oq, os_ = Q.mx_quant_rowwise(xf, fmt)
    assert np.array_equal(codes_np(rs), os_) and np.array_equal(codes_np(rq), oq)
    oq, os_ = Q.mx_quant_colwise(xf, fmt)
    assert np.array_equal(codes_np(cs), os_) and np.array_equal(codes_np(cq), oq)
    assert codes_np(rs)[8:, :].max() == 0  # untouched rows: all-zero blocks
    q1, s1 = _fn(fmt)(xb.cuda(), dt, 1, 32)  # the row direction alone: same bytes
    assert torch.equal(q1.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(s1.view(torch.uint8), rs.view(torch.uint8))


@pytest.mark.parametrize("fmt,dt", FMTS)
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_mx_dequant_matches_oracle(fmt, dt, out_dtype):
    x = bf16_randn((200, 160), seed=54, outlier_frac=0.01).cuda()
    rq, rs, cq, cs = _fn(fmt)(x, dt, None, 32, with_trans=True)
    y = _dq(fmt)(rq, out_dtype, 1, 32, rs)
    ref = torch.from_numpy(Q.mx_dequant(codes_np(rq), codes_np(rs), fmt)).to(out_dtype)
    assert torch.equal(y.cpu(), ref)
    yt = _dq(fmt)(cq, out_dtype, 0, 32, cs)  # transposed back: [M_pad, N]
    ref_t = torch.from_numpy(np.ascontiguousarray(Q.mx_dequant(codes_np(cq), codes_np(cs), fmt).T)).to(out_dtype)
    assert torch.equal(yt.cpu(), ref_t)
    # round trip stays within half a code step of the block scale
    err = (y[:, :160].float() - x.float()).abs().max().item()
    # (relative code spacing: E2M1 1/2, E5M2 1/4, E4M3 1/8; the top sliver of a block saturates)
    assert err <= x.float().abs().max().item() * {"e2m1": 0.26, "e5m2": 0.14, "e4m3": 0.07}[fmt]


def test_mx_public_ops():
    """The public quantize_fp8 / quantize_fp4 entry points route MX_BLOCKWISE to these kernels."""
    x = bf16_randn((256, 256), seed=55).cuda()
    q, s = turbo.ops.quantize_fp8(x, torch.float8_e4m3fn, G.MX_BLOCKWISE, block_size=32, axis=1)
    oq, os_ = Q.mx_quant_rowwise(to_f32_np(x), "e4m3")
    assert np.array_equal(codes_np(q), oq) and np.array_equal(codes_np(s), os_)
    y = turbo.ops.dequantize_fp8(q, torch.bfloat16, G.MX_BLOCKWISE, block_size=32, axis=1, scale_inv=s)
    assert torch.equal(y.cpu(), torch.from_numpy(Q.mx_dequant(oq, os_, "e4m3")).to(torch.bfloat16))
    if FP4 is not None:
        q, s = turbo.ops.quantize_fp4(x, FP4, G.MX_BLOCKWISE, block_size=32, axis=1)
        oq, os_ = Q.mx_quant_rowwise(to_f32_np(x), "e2m1")
        assert np.array_equal(codes_np(q), oq) and np.array_equal(codes_np(s), os_)


@pytest.mark.skipif(FP4 is None, reason="torch has no float4_e2m1fn_x2")
@pytest.mark.parametrize("row_rht,col_rht", [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize("M,N", [(128, 128), (200, 96), (33, 32), (1000, 2080), (4096, 1024)])
def test_mxfp4_hadamard_recipe_matches_oracle(row_rht, col_rht, M, N):
    """``use_rht``: codes and scale bytes of the Hadamard-transformed values, per direction (the recipe
    uses it on the column direction of ``a`` and ``grad_out``; padding rows / columns take part as
    zeros). Dual call, single-direction calls, fp16 input."""
    x = bf16_randn((M, N), seed=55, outlier_frac=0.002)
    r, rt = ScalingRecipe(use_rht=row_rht), ScalingRecipe(use_rht=col_rht)
    rq, rs, cq, cs = qi.quantize_mxfp4_impl(x.cuda(), FP4, None, 32, with_trans=True, scaling_recipe=r,
                                            scaling_recipe_for_trans=rt)
    xf = to_f32_np(x)
    oq, os_ = Q.mx_quant_rowwise(xf, "e2m1", use_rht=row_rht)
    assert np.array_equal(codes_np(rs), os_) and np.array_equal(codes_np(rq), oq), "row direction"
    oq, os_ = Q.mx_quant_colwise(xf, "e2m1", use_rht=col_rht)
    assert np.array_equal(codes_np(cs), os_) and np.array_equal(codes_np(cq), oq), "column direction"
    q0, s0 = qi.quantize_mxfp4_impl(x.cuda(), FP4, 0, 32, scaling_recipe=rt)
    assert torch.equal(q0.view(torch.uint8), cq.view(torch.uint8)) and torch.equal(s0.view(torch.uint8), cs.view(torch.uint8))
    q1, s1 = qi.quantize_mxfp4_impl(x.cuda(), FP4, 1, 32, scaling_recipe=r)
    assert torch.equal(q1.view(torch.uint8), rq.view(torch.uint8)) and torch.equal(s1.view(torch.uint8), rs.view(torch.uint8))
    xh = x.to(torch.float16)
    hq, hs = qi.quantize_mxfp4_impl(xh.cuda(), FP4, 0, 32, scaling_recipe=ScalingRecipe(use_rht=True))
    oq, os_ = Q.mx_quant_colwise(to_f32_np(xh), "e2m1", use_rht=True)
    assert np.array_equal(codes_np(hs), os_) and np.array_equal(codes_np(hq), oq), "fp16 input"


@pytest.mark.skipif(FP4 is None, reason="torch has no float4_e2m1fn_x2")
def test_mx_hadamard_recipe_limits():
    x = bf16_randn((128, 128), seed=56).cuda()
    with pytest.raises(NotImplementedError):  # MXFP8 has no Hadamard recipe
        qi.quantize_mxfp8_impl(x, torch.float8_e4m3fn, 1, 32, scaling_recipe=ScalingRecipe(use_rht=True))
    with pytest.raises(NotImplementedError):  # never together with 2-D blocks
        qi.quantize_mxfp4_impl(x, FP4, 1, 32, scaling_recipe=ScalingRecipe(use_rht=True, use_2d_block=True))
    with pytest.raises(NotImplementedError):  # MXFP8 has no stochastic rounding either
        qi.quantize_mxfp8_impl(x, torch.float8_e4m3fn, 1, 32, scaling_recipe=ScalingRecipe(use_sr=True))
    with pytest.raises(RuntimeError, match="divisible by 16"):  # shuffled codes come in bands of 16 rows
        qi.quantize_mxfp4_impl(x[:120].contiguous(), FP4, 1, 32, scaling_recipe=ScalingRecipe(shuffle_out=True))


@pytest.mark.skipif(FP4 is None, reason="torch has no float4_e2m1fn_x2")
@pytest.mark.parametrize("axis", [1, 0])
@pytest.mark.parametrize("rht", [False, True])
def test_mxfp4_stochastic_rounding(axis, rht):
    """``use_sr``: the scale bytes are those of round-to-nearest; every code is one of the two E2M1
    neighbours of the scaled value; two calls differ (fresh seed) yet the mean over many calls
    converges to the unrounded value (unbiased) where round-to-nearest keeps its systematic error."""
    M, N = 256, 128
    x = bf16_randn((M, N), seed=57)
    xf = to_f32_np(x)
    plain = ScalingRecipe(use_rht=rht)
    q0, s0 = qi.quantize_mxfp4_impl(x.cuda(), FP4, axis, 32, scaling_recipe=plain)
    rec = ScalingRecipe(use_sr=True, use_rht=rht)
    n_calls = 192
    acc = None
    codes = []
    for _ in range(n_calls):
        q, sc = qi.quantize_mxfp4_impl(x.cuda(), FP4, axis, 32, scaling_recipe=rec)
        assert torch.equal(sc.view(torch.uint8), s0.view(torch.uint8)), "scales are deterministic"
        d = Q.mx_dequant(codes_np(q), codes_np(sc), "e2m1").astype(np.float64)
        acc = d if acc is None else acc + d
        if len(codes) < 2:
            codes.append(codes_np(q).copy())
    assert not np.array_equal(codes[0], codes[1]), "a fresh seed per call"
    # the exact values the codes approximate: the (transformed) tensor in the quantizer's layout
    t = xf if axis == 1 else np.ascontiguousarray(xf.T)
    pad = np.zeros((t.shape[0], -(-t.shape[1] // 128) * 128), np.float32)
    pad[:, : t.shape[1]] = t
    target = (Q.hadamard16(pad) if rht else pad).astype(np.float64)
    scale = np.repeat(Q.e8m0_to_f32(codes_np(s0)).astype(np.float64), 32, axis=-1)
    grid = np.array([0, .5, 1, 1.5, 2, 3, 4, 6], dtype=np.float64)
    # each code is a neighbour of the clamped scaled value
    one = Q.mx_dequant(codes[0], codes_np(s0), "e2m1").astype(np.float64) / scale
    v = np.clip(target / scale, -6, 6)
    lo = grid[np.searchsorted(grid, np.abs(v), side="right") - 1]
    hi = grid[np.minimum(np.searchsorted(grid, np.abs(v), side="left"), 7)]
    assert np.all((np.abs(one) == lo) | (np.abs(one) == hi))
    # unbiased: the mean error shrinks like 1 / sqrt(n), far below round-to-nearest's
    mean = acc / n_calls
    inside = np.abs(target / scale) <= 6  # the saturated sliver of a block is clamped, not rounded
    err_sr = np.abs(mean - target)[inside] / scale[inside]
    rne = Q.mx_dequant(codes_np(q0), codes_np(s0), "e2m1").astype(np.float64)
    err_rne = np.abs(rne - target)[inside] / scale[inside]
    assert err_sr.mean() < 0.35 * err_rne.mean(), (err_sr.mean(), err_rne.mean())
    assert err_sr.max() < 6 * 1.0 / np.sqrt(n_calls) + 1e-6  # within six standard errors of the largest step
