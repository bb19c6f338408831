"""The reference's MX dispatcher operators called by their own names
(``torch.ops.primus_turbo_cpp_extension.*``; schemas of csrc/pytorch/bindings_pytorch.cpp:44,52-93):
outputs bit-exact against the CPU oracle, shapes as csrc/pytorch/quantization/quantization.cpp
states them, and the Meta implementations agree with the device ones on shapes and dtypes."""

import numpy as np
import pytest
import torch

from helpers import bf16_randn, codes_np, group_lens, to_f32_np
from oracle import quantize as Q

pytestmark = pytest.mark.gpu

F4 = getattr(torch, "float4_e2m1fn_x2", None)
E8 = getattr(torch, "float8_e8m0fnu", torch.uint8)


@pytest.fixture(scope="module", autouse=True)
def _ext(native_lib):
    global ext, Qi
    import primus_turbo.pytorch  # noqa: F401  (registers the operators)
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as Qi

    ext = torch.ops.primus_turbo_cpp_extension


def _same_meta(op, args, outs):
    metas = op(*[a.to("meta") if isinstance(a, torch.Tensor) else a for a in args])
    metas = metas if isinstance(metas, (list, tuple)) else [metas]
    outs = outs if isinstance(outs, (list, tuple)) else [outs]
    assert len(metas) == len(outs)
    for m, o in zip(metas, outs):
        assert tuple(m.shape) == tuple(o.shape) and m.dtype == o.dtype, (m.shape, o.shape, m.dtype, o.dtype)


@pytest.mark.parametrize("fmt,dt", [("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)])
@pytest.mark.parametrize("use_2d", [False, True])
def test_quantize_mxfp8_and_dual_and_dequantize(fmt, dt, use_2d):
    x = bf16_randn((200, 320), seed=71, outlier_frac=0.001).cuda()
    xf = to_f32_np(x)
    oq, os_ = Q.mx_quant_rowwise(xf, fmt, use_2d_block=use_2d)
    cq, cs = Q.mx_quant_colwise(xf, fmt, use_2d_block=use_2d)
    q, s = ext.quantize_mxfp8(x, dt, 1, 128, use_2d)
    assert q.dtype == dt and s.dtype == E8 and tuple(q.shape) == (200, 384) and tuple(s.shape) == (200, 12)
    assert np.array_equal(codes_np(q), oq) and np.array_equal(codes_np(s), os_)
    _same_meta(ext.quantize_mxfp8, (x, dt, 1, 128, use_2d), [q, s])
    q0, s0 = ext.quantize_mxfp8(x, dt, 0, 128, use_2d)
    assert tuple(q0.shape) == (320, 256) and np.array_equal(codes_np(q0), cq) and np.array_equal(codes_np(s0), cs)
    _same_meta(ext.quantize_mxfp8, (x, dt, 0, 128, use_2d), [q0, s0])
    outs = ext.quantize_mxfp8_dual(x, dt, 128, use_2d, use_2d)
    assert len(outs) == 4
    for got, want in zip(outs, (oq, os_, cq, cs)):
        assert np.array_equal(codes_np(got), want)
    _same_meta(ext.quantize_mxfp8_dual, (x, dt, 128, use_2d, use_2d), outs)
    # de-quantize both directions back (the column direction comes back transposed: [M_pad, N])
    y = ext.dequantize_mxfp8(q, s, 1, 32, torch.bfloat16)
    want = torch.from_numpy(Q.mx_dequant(oq, os_, fmt)).to(torch.bfloat16)
    assert torch.equal(y.cpu(), want)
    _same_meta(ext.dequantize_mxfp8, (q, s, 1, 32, torch.bfloat16), y)
    y0 = ext.dequantize_mxfp8(q0, s0, 0, 32, torch.float32)
    want0 = torch.from_numpy(np.ascontiguousarray(Q.mx_dequant(cq, cs, fmt).T))
    assert torch.equal(y0.cpu(), want0)
    _same_meta(ext.dequantize_mxfp8, (q0, s0, 0, 32, torch.float32), y0)
    with pytest.raises((RuntimeError, NotImplementedError)):
        ext.quantize_mxfp8(x, dt, 1, 64, use_2d)  # only the 128 padding exists
    with pytest.raises(RuntimeError):
        ext.quantize_mxfp8(x, dt, 2, 128, use_2d)


@pytest.mark.skipif(F4 is None, reason="torch without float4_e2m1fn_x2")
def test_quantize_mxfp4_and_dual_and_dequantize():
    x = bf16_randn((96, 256), seed=72).cuda()
    xf = to_f32_np(x)
    oq, os_ = Q.mx_quant_rowwise(xf, "e2m1")
    cq, cs = Q.mx_quant_colwise(xf, "e2m1", use_2d_block=True)
    q, s = ext.quantize_mxfp4(x, F4, 1, 128, False, False, False)
    assert q.dtype == F4 and tuple(q.shape) == (96, 128) and tuple(s.shape) == (96, 8)
    assert np.array_equal(codes_np(q), oq) and np.array_equal(codes_np(s), os_)
    _same_meta(ext.quantize_mxfp4, (x, F4, 1, 128, False, False, False), [q, s])
    outs = ext.quantize_mxfp4_dual(x, F4, 128, False, False, False, True, False, False)
    for got, want in zip(outs, (oq, os_, cq, cs)):
        assert np.array_equal(codes_np(got), want)
    _same_meta(ext.quantize_mxfp4_dual, (x, F4, 128, False, False, False, True, False, False), outs)
    y = ext.dequantize_mxfp4(q, s, 1, 32, torch.float32)
    assert torch.equal(y.cpu(), torch.from_numpy(Q.mx_dequant(oq, os_, "e2m1")))
    _same_meta(ext.dequantize_mxfp4, (q, s, 1, 32, torch.float32), y)
    # the Hadamard recipe goes through the same operator
    hq, hs = ext.quantize_mxfp4(x, F4, 1, 128, False, False, True)
    rq, rs = Q.mx_quant_rowwise(xf, "e2m1", use_rht=True)
    assert np.array_equal(codes_np(hq), rq) and np.array_equal(codes_np(hs), rs)


def test_meta_shapes_with_shuffled_scales():
    """shuffle_scale pads the scale of every matrix (rows to 256, columns to 8): the Meta
    implementations have to say so too, also for 3-D input and where M is no multiple of 256."""
    for shape in ((200, 320), (3, 136, 160)):
        x = bf16_randn(shape, seed=73).cuda()
        dt = torch.float8_e4m3fn
        for axis in (x.dim() - 1, x.dim() - 2):
            args = (x, dt, axis, 128, False, True, False)
            outs = ext.quantize_mxfp8(*args)
            assert tuple(outs[1].shape[-2:]) == Qi._scale_pad(*outs[1].shape[-2:])  # padded already
            _same_meta(ext.quantize_mxfp8, args, outs)
        for flags in ((True, False, False, False), (False, False, True, False), (True, False, True, False)):
            args = (x, dt, 128, False, False) + flags
            _same_meta(ext.quantize_mxfp8_dual, args, ext.quantize_mxfp8_dual(*args))
        if F4 is not None:
            args = (x, F4, x.dim() - 1, 128, False, False, False, True, False)
            _same_meta(ext.quantize_mxfp4, args, ext.quantize_mxfp4(*args))
            args = (x, F4, 128, False, False, False, False, False, False, True, False, True, False)
            _same_meta(ext.quantize_mxfp4_dual, args, ext.quantize_mxfp4_dual(*args))


def test_grouped_quantize_mxfp8_names():
    G_, M, N = 6, 700, 256
    lens = group_lens("ragged", G_, M, 73)
    lens[2] = 0
    lens[-1] += M - lens.sum()
    gl = torch.from_numpy(lens).cuda()
    offs = ext.grouped_gemm_compute_offs(gl)
    x = bf16_randn((M, N), seed=74).cuda()
    want = Q.mx_grouped_quant(to_f32_np(x), lens, "e4m3")
    dt = torch.float8_e4m3fn
    outs = ext.grouped_quantize_mxfp8_dual(x, gl, offs, dt, False, False)
    assert len(outs) == 8
    rq, rs, cq, cs, lr, orow, lc, ocol = outs
    offs_r, offs_c = orow.cpu().numpy(), ocol.cpu().numpy()
    assert np.array_equal(offs_r, want["row_offs"]) and np.array_equal(offs_c, want["col_offs"])
    nr, nc = int(offs_r[-1]), int(offs_c[-1])
    assert np.array_equal(codes_np(rq)[:nr], want["row"][:nr]) and np.array_equal(codes_np(rs)[:nr], want["row_scale"][:nr])
    assert np.array_equal(codes_np(cq)[:, :nc], want["col"][:, :nc])
    assert np.array_equal(codes_np(cs)[:, : nc // 32], want["col_scale"][:, : nc // 32])
    _same_meta(ext.grouped_quantize_mxfp8_dual, (x, gl, offs, dt, False, False), outs)
    one = ext.grouped_quantize_mxfp8(x, gl, offs, dt, 1, 128, False)
    assert len(one) == 4 and torch.equal(one[0].view(torch.uint8)[:nr], rq.view(torch.uint8)[:nr])
    _same_meta(ext.grouped_quantize_mxfp8, (x, gl, offs, dt, 1, 128, False), one)
    zero = ext.grouped_quantize_mxfp8(x, gl, offs, dt, 0, 128, False)
    assert torch.equal(zero[0].view(torch.uint8)[:, :nc], cq.view(torch.uint8)[:, :nc])
    # and back: packed rows from the padded layout
    y = ext.grouped_dequantize_mxfp8(rq, rs, offs, orow, 1, 32, torch.float32, M)
    ref = Q.mx_dequant(want["row"], want["row_scale"], "e4m3")
    src = np.concatenate([np.arange(lens[g]) + offs_r[g] for g in range(G_)]).astype(np.int64)
    assert np.array_equal(y.cpu().numpy(), ref[src][:, :N])
    _same_meta(ext.grouped_dequantize_mxfp8, (rq, rs, offs, orow, 1, 32, torch.float32, M), y)
    # 2-D blocks and the pre-shuffled forms, by the reference's argument names
    want2 = Q.mx_grouped_quant(to_f32_np(x), lens, "e4m3", row_2d=True, col_2d=True)
    two = ext.grouped_quantize_mxfp8(x, gl, offs, dt, 1, 128, True)
    assert np.array_equal(codes_np(two[0])[:nr], want2["row"][:nr]) and np.array_equal(codes_np(two[1])[:nr], want2["row_scale"][:nr])
    _same_meta(ext.grouped_quantize_mxfp8, (x, gl, offs, dt, 1, 128, True), two)
    shuf = ext.grouped_quantize_mxfp8_dual(x, gl, offs, dt, False, True, True, True, True, False)
    back, sback = Qi.mx_plain_layout(shuf[0], shuf[1], True, True)
    assert torch.equal(back.view(torch.uint8)[:nr], rq.view(torch.uint8)[:nr])
    assert torch.equal(sback.view(torch.uint8)[:nr], rs.view(torch.uint8)[:nr])
    assert np.array_equal(codes_np(shuf[2])[:, :nc], want2["col"][:, :nc])  # column codes: 2-D blocks, not shuffled
    assert np.array_equal(codes_np(ext.unshuffle_scale(shuf[3], cs.shape[0], cs.shape[1]))[:, : nc // 32],
                          want2["col_scale"][:, : nc // 32])
    _same_meta(ext.grouped_quantize_mxfp8_dual, (x, gl, offs, dt, False, True, True, True, True, False), shuf)


@pytest.mark.skipif(F4 is None, reason="torch without float4_e2m1fn_x2")
def test_grouped_quantize_mxfp4_names():
    G_, M, N = 4, 512, 256
    lens = group_lens("ragged", G_, M, 75)
    gl = torch.from_numpy(lens).cuda()
    offs = ext.grouped_gemm_compute_offs(gl)
    x = bf16_randn((M, N), seed=76).cuda()
    outs = ext.grouped_quantize_mxfp4_dual(x, gl, offs, F4, False, False, False, False, False, False)
    assert len(outs) == 8
    oq, os_ = Q.mx_quant_rowwise(to_f32_np(x), "e2m1")
    assert np.array_equal(codes_np(outs[0]), oq) and np.array_equal(codes_np(outs[1]), os_)
    assert torch.equal(outs[4], gl) and torch.equal(outs[5], offs)  # the row direction keeps the tight layout
    _same_meta(ext.grouped_quantize_mxfp4_dual, (x, gl, offs, F4, False, False, False, False, False, False), outs)
    row = ext.grouped_quantize_mxfp4(x, gl, offs, F4, 1, False, False, False)
    assert len(row) == 4 and np.array_equal(codes_np(row[0]), oq)
    col = ext.grouped_quantize_mxfp4(x, gl, offs, F4, 0, False, False, False)
    nc = int(outs[7][-1].item())  # what lies beyond the last group's padded columns is unspecified
    assert torch.equal(col[0].view(torch.uint8)[:, : nc // 2], outs[2].view(torch.uint8)[:, : nc // 2])
    assert torch.equal(col[3], outs[7])


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.uint8, torch.bfloat16, torch.float32, torch.int64])
@pytest.mark.parametrize("shape", [(130, 70), (3, 65, 129), (1, 1), (0, 5)])
def test_transpose_2d(dtype, shape):
    g = torch.Generator().manual_seed(77)
    raw = torch.randint(0, 255, shape, generator=g, dtype=torch.uint8)
    x = (raw.to(dtype) if dtype != torch.float8_e4m3fn else raw.view(dtype)).cuda().contiguous()
    y = ext.transpose_2d(x, -1, -2)
    want = x.view(torch.uint8).cpu() if dtype == torch.float8_e4m3fn else x.cpu()
    got = y.view(torch.uint8).cpu() if dtype == torch.float8_e4m3fn else y.cpu()
    assert y.is_contiguous() and torch.equal(got, want.transpose(-1, -2))
    _same_meta(ext.transpose_2d, (x, -1, -2), y)
    nd = len(shape)
    assert torch.equal(ext.transpose_2d(x, nd - 2, nd - 1).view(torch.uint8), y.view(torch.uint8))
    if nd == 3:
        with pytest.raises(RuntimeError, match="last two dims"):
            ext.transpose_2d(x, 0, 1)
