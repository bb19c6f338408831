"""The hot path under HIP graph capture (``torch.cuda.graph``): quantize -> GEMM steps, grouped
forward + backward, are captured once and replayed with new contents in the static input buffers;
every replay must equal the eager result bit for bit, with eager work and synchronizations between
the replays (the reference captures its grouped MXFP4 GEMM the same way,
tests/pytorch/ops/test_grouped_gemm_fp4.py:409-470). One eager call before the capture does the
one-time set-up (kernel attributes, lazy library loading) outside the graph."""

import pytest
import torch

from helpers import bf16_randn, group_lens

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, G, F8, F4, Format, ScaleDtype
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import Float4QuantConfig as F4
    from primus_turbo.pytorch.core.low_precision import Float8QuantConfig as F8
    from primus_turbo.pytorch.core.low_precision import Format, ScaleDtype
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G


def _replay_check(fn, make_inputs, n_static, replays=3):
    """``fn(*static) -> tuple of tensors``; ``make_inputs(seed) -> tuple`` of fresh CPU-made inputs."""
    static = [t.cuda() for t in make_inputs(0)]
    assert len(static) == n_static
    fn(*static)  # one-time set-up outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn(*static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = fn(*static)
    for seed in range(1, replays + 1):
        fresh = [t.cuda() for t in make_inputs(seed)]
        for s, f in zip(static, fresh):
            s.copy_(f)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = fn(*fresh)  # eager work between the replays
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g.view(torch.uint8) if g.element_size() == 1 else g,
                               w.view(torch.uint8) if w.element_size() == 1 else w), f"replay {seed} differs from eager"


def test_graph_tensorwise_quantize_dequantize():
    def fn(x):
        q, s = turbo.ops.quantize_fp8(x, turbo.float8_e4m3, G.TENSORWISE)
        return q, s, turbo.ops.dequantize_fp8(q, torch.bfloat16, G.TENSORWISE, scale_inv=s)

    _replay_check(fn, lambda seed: (bf16_randn((1024, 1024), seed=100 + seed, outlier_frac=0.001) * (1 + seed),), 1)


def test_two_graphs_on_the_capture_stream_tensorwise():
    """Two graphs captured one after the other on torch's capture stream, each holding a dynamic
    tensorwise quantizer, replayed in order (and the first again): neither may see the other's
    abs-max. Nothing of a captured quantizer lives in per-stream state of the library."""
    import numpy as np

    from helpers import bits_np, codes_np, to_f32_np
    from oracle import quantize as Q

    xa = bf16_randn((1024, 1024), seed=170, outlier_frac=0.001).cuda()
    xb = (bf16_randn((512, 2048), seed=171) * 37.0).cuda()
    turbo.ops.quantize_fp8(xa, turbo.float8_e4m3, G.TENSORWISE)  # one-time set-up outside the captures
    torch.cuda.synchronize()
    ga, gb = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
    with torch.cuda.graph(ga):
        qa, sa = turbo.ops.quantize_fp8(xa, turbo.float8_e4m3, G.TENSORWISE)
    with torch.cuda.graph(gb):
        qb, sb = turbo.ops.quantize_fp8(xb, turbo.float8_e4m3, G.TENSORWISE)
    for rep in range(3):
        xa.mul_(1.5)
        ga.replay()
        gb.replay()
        turbo.ops.quantize_fp8(xb, turbo.float8_e4m3, G.TENSORWISE)  # eager work on the same stream
        ga.replay()
        torch.cuda.synchronize()
        for x, q, s in ((xa, qa, sa), (xb, qb, sb)):
            oq, osinv = Q.fp8_tensorwise(to_f32_np(x.cpu()), "e4m3")
            assert bits_np(s).item() == osinv.view(np.uint32).item(), rep
            assert np.array_equal(codes_np(q), oq), rep


@pytest.mark.parametrize("gran", ["ROWWISE", "BLOCKWISE", "MX_BLOCKWISE"])
def test_graph_gemm_fp8_forward(gran):
    kw = {"BLOCKWISE": dict(block_size=128), "MX_BLOCKWISE": dict(block_size=32, scale_dtype=ScaleDtype.E8M0)}.get(gran, {})
    cfg = F8(format=Format.E4M3, granularity=getattr(G, gran), **kw)

    def fn(a, b):
        return (turbo.ops.gemm_fp8(a, b, trans_b=True, config=cfg),)

    _replay_check(fn, lambda seed: (bf16_randn((512, 1024), seed=110 + seed), bf16_randn((768, 1024), seed=120 + seed)), 2)


@pytest.mark.parametrize("kind", ["blockwise", "mxfp8", "mxfp4"])
def test_graph_grouped_gemm_forward_backward(kind):
    lens = group_lens("ragged", 4, 1024, 130)
    gl = torch.from_numpy(lens).cuda()
    if kind == "mxfp4":
        cfg, op = F4(), turbo.ops.grouped_gemm_fp4
    else:
        kw = dict(block_size=128) if kind == "blockwise" else dict(block_size=32, scale_dtype=ScaleDtype.E8M0)
        cfg = F8(format=Format.E4M3, granularity=G.BLOCKWISE if kind == "blockwise" else G.MX_BLOCKWISE, **kw)
        op = turbo.ops.grouped_gemm_fp8

    def fn(a, b, dy):
        a = a.detach().requires_grad_(True)
        b = b.detach().requires_grad_(True)
        y = op(a, b, gl, trans_b=True, config=cfg)
        da, db = torch.autograd.grad(y, (a, b), dy)
        return y, da, db

    _replay_check(fn, lambda seed: (bf16_randn((1024, 1024), seed=140 + seed), bf16_randn((4, 512, 1024), seed=150 + seed),
                                    bf16_randn((1024, 512), seed=160 + seed)), 3)


@pytest.mark.parametrize("kind", ["blockwise", "mxfp8", "mxfp4"])
def test_graph_grouped_gemm_replays_with_other_group_lens(kind):
    """The grouped kernels look their groups up on the device, so one captured graph serves any
    split of the same token count: the static ``group_lens`` tensor is rewritten between replays
    (another split, then one with an expert going empty, then the first again) and every replay
    must equal the eager result for that split bit for bit, forward and backward (the reference
    holds this test, skipped there: tests/pytorch/ops/test_grouped_gemm_fp8.py:1029)."""
    import numpy as np

    M, Gn = 1024, 4
    splits = [group_lens("ragged", Gn, M, 131), group_lens("ragged", Gn, M, 977), np.array([700, 0, 24, 300], dtype=np.int64),
              np.array([1, 1021, 1, 1], dtype=np.int64)]
    assert all(int(x.sum()) == M for x in splits)
    if kind == "mxfp4":
        cfg, op = F4(), turbo.ops.grouped_gemm_fp4
    else:
        kw = dict(block_size=128) if kind == "blockwise" else dict(block_size=32, scale_dtype=ScaleDtype.E8M0)
        cfg = F8(format=Format.E4M3, granularity=G.BLOCKWISE if kind == "blockwise" else G.MX_BLOCKWISE, **kw)
        op = turbo.ops.grouped_gemm_fp8

    def fn(a, b, dy, gl):
        a = a.detach().requires_grad_(True)
        b = b.detach().requires_grad_(True)
        y = op(a, b, gl, trans_b=True, config=cfg)
        da, db = torch.autograd.grad(y, (a, b), dy)
        return y, da, db

    def make(seed):
        return (bf16_randn((M, 1024), seed=180 + seed), bf16_randn((Gn, 512, 1024), seed=190 + seed),
                bf16_randn((M, 512), seed=200 + seed), torch.from_numpy(splits[seed % len(splits)]))

    _replay_check(fn, make, 4, replays=5)


def test_stochastic_rounding_refuses_graph_capture():
    """The stochastic-rounding seed is a host-side launch argument: captured, every replay would
    round with the same noise. The quantizer raises under capture instead (and works outside)."""
    F4 = getattr(torch, "float4_e2m1fn_x2", None)
    if F4 is None:
        pytest.skip("torch without float4_e2m1fn_x2")
    from primus_turbo.pytorch.core.low_precision import ScalingRecipe
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

    x = bf16_randn((128, 256), seed=3).cuda()
    sr = ScalingRecipe(use_sr=True)
    qi.quantize_mxfp4_impl(x, F4, 1, 32, False, sr)  # eager: fine
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="cannot be captured"):
        with torch.cuda.graph(graph, stream=side):
            qi.quantize_mxfp4_impl(x, F4, 1, 32, False, sr)
    torch.cuda.synchronize()
    # round-to-nearest captures as before
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2):
        q, s = qi.quantize_mxfp4_impl(x, F4, 1, 32, False, ScalingRecipe())
    g2.replay()
    torch.cuda.synchronize()
    q0, s0 = qi.quantize_mxfp4_impl(x, F4, 1, 32, False, ScalingRecipe())
    assert torch.equal(q.view(torch.uint8), q0.view(torch.uint8)) and torch.equal(s.view(torch.uint8), s0.view(torch.uint8))
