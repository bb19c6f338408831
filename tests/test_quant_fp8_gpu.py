"""GPU parity: tensorwise / rowwise FP8 quantize + dequantize vs the CPU oracle (bit-exact)."""

import numpy as np
import pytest
import torch

from helpers import FMT, bf16_randn, bits_np, codes_np, round_to, to_f32_np
from oracle import quantize as Q

pytestmark = pytest.mark.gpu

G = None


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global G, turbo
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity

    G = ScalingGranularity


def _check_tensorwise(x, dtype):
    q, sinv = turbo.ops.quantize_fp8(x.cuda(), dtype, G.TENSORWISE)
    torch.cuda.synchronize()
    oq, osinv = Q.fp8_tensorwise(to_f32_np(x), FMT[dtype])
    assert q.dtype == dtype and q.shape == x.shape and sinv.shape == ()
    assert bits_np(sinv).item() == osinv.view(np.uint32).item(), (sinv.item(), osinv.item())
    got = codes_np(q)
    assert np.array_equal(got, oq), f"{(got != oq).sum()} of {got.size} bytes differ"
    return q, sinv


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("src", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(4096, 4096), (333, 257), (1,), (15,), (16,), (17,), (2880,), (2881,), (5, 7, 64)])
def test_tensorwise_bit_exact(shape, src, dtype):
    if shape == (4096, 4096) and src != torch.bfloat16:
        pytest.skip("headline size only for bf16")
    x = bf16_randn(shape, seed=0, outlier_frac=0.001, dtype=src)
    q, sinv = _check_tensorwise(x, dtype)
    # dequantize: y = T(float(q) * scale_inv)
    y = turbo.ops.dequantize_fp8(q, src, G.TENSORWISE, scale_inv=sinv)
    torch.cuda.synchronize()
    oy = round_to(Q.fp8_dequant(codes_np(q), to_f32_np(sinv), FMT[dtype]), src)
    assert y.dtype == src
    assert np.array_equal(bits_np(y), bits_np(oy))


def test_tensorwise_special_values():
    # all zero: scale = 448 / 1e-12
    x = torch.zeros(1000, dtype=torch.bfloat16)
    q, sinv = _check_tensorwise(x, torch.float8_e4m3fn)
    assert codes_np(q).max() == 0
    # a single spike among small values
    x = torch.full((4096 * 3 + 5,), 1e-3, dtype=torch.bfloat16)
    x[7777] = -300.0
    _check_tensorwise(x, torch.float8_e4m3fn)
    # NaN maps to +max, inf gives scale 0 (finite values -> 0, inf * 0 = NaN -> +max)
    x = bf16_randn((4096,), 3)
    x[5] = float("nan")
    _check_tensorwise(x, torch.float8_e4m3fn)
    x[9] = float("inf")
    _check_tensorwise(x, torch.float8_e4m3fn)
    # large tensor beyond what the registers park (re-read path) and a ragged tail
    x = bf16_randn((256 * 1024 * 16 * 5 + 3,), 4)
    _check_tensorwise(x, torch.float8_e5m2)


def test_tensorwise_unaligned_matches_aligned():
    base = bf16_randn((4096 * 8 + 16,), 5, outlier_frac=0.01)
    for off in (0, 1, 3, 8):
        x = base[off : off + 4096 * 8]
        assert x.is_contiguous()
        xg = base.cuda()[off : off + 4096 * 8]
        q, sinv = turbo.ops.quantize_fp8(xg, torch.float8_e4m3fn, G.TENSORWISE)
        oq, osinv = Q.fp8_tensorwise(to_f32_np(x), "e4m3")
        assert np.array_equal(codes_np(q), oq)
        assert bits_np(sinv).item() == osinv.view(np.uint32).item()


def test_tensorwise_repeat_calls_reuse_workspace():
    # the kernel must leave its workspace zeroed: a large-amax call followed by a small one
    big = bf16_randn((1 << 20,), 6, scale=100.0)
    small = bf16_randn((1 << 16,), 7, scale=0.01)
    for x in (big, small, big, small):
        _check_tensorwise(x, torch.float8_e4m3fn)


def test_tensorwise_given_scale():
    x = bf16_randn((1000, 100), 8)
    scale = torch.tensor(3.7, dtype=torch.float32)
    q, sinv = torch.ops.primus_turbo_cpp_extension.quantize_fp8_tensorwise(x.cuda(), torch.float8_e4m3fn, scale.cuda())
    oq, osinv = Q.fp8_tensorwise(to_f32_np(x), "e4m3", scale=scale.numpy())
    assert np.array_equal(codes_np(q), oq)
    assert bits_np(sinv).item() == osinv.view(np.uint32).item()


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize(
    "shape,axis",
    [
        ((8192, 8192), -1),
        ((512, 8192), 0),
        ((4, 111, 4096), -1),
        ((4, 111, 4096), 1),
        ((4, 111, 4096), 0),
        ((1, 1, 1), 2),
        ((3, 111, 111), -2),
        ((7168, 111), 1),
        ((2, 40000), -1),
        ((64, 24), 1),
    ],
)
def test_rowwise_bit_exact(shape, axis, dtype):
    if shape[0] == 8192 and dtype != torch.float8_e4m3fn:
        pytest.skip("headline size only for e4m3")
    x = bf16_randn(shape, seed=11, scale=0.02 if shape[0] == 8192 else 1.0, outlier_frac=0.001)
    q, sinv = turbo.ops.quantize_fp8(x.cuda(), dtype, G.ROWWISE, axis=axis)
    torch.cuda.synchronize()
    oq, osinv = Q.fp8_rowwise(to_f32_np(x), axis, FMT[dtype])
    assert tuple(sinv.shape) == osinv.shape
    assert np.array_equal(bits_np(sinv), osinv.view(np.uint32))
    assert np.array_equal(codes_np(q), oq)
    y = turbo.ops.dequantize_fp8(q, torch.bfloat16, G.ROWWISE, axis=axis, scale_inv=sinv)
    oy = round_to(Q.fp8_dequant(oq, osinv, FMT[dtype]), torch.bfloat16)
    assert np.array_equal(bits_np(y), bits_np(oy))


@pytest.mark.parametrize("src", [torch.float16, torch.float32])
def test_rowwise_other_sources(src):
    x = bf16_randn((37, 1000), 12, dtype=src)
    for axis in (0, 1):
        q, sinv = turbo.ops.quantize_fp8(x.cuda(), torch.float8_e4m3fn, G.ROWWISE, axis=axis)
        oq, osinv = Q.fp8_rowwise(to_f32_np(x), axis, "e4m3")
        assert np.array_equal(codes_np(q), oq)
        assert np.array_equal(bits_np(sinv), osinv.view(np.uint32))
        y = turbo.ops.dequantize_fp8(q, src, G.ROWWISE, axis=axis, scale_inv=sinv)
        assert np.array_equal(bits_np(y), bits_np(round_to(Q.fp8_dequant(oq, osinv, "e4m3"), src)))


def test_literal_python_reference_within_its_tolerance():
    # the reference's own test tolerance vs its pure-PyTorch formula
    # (tests/pytorch/ops/test_quantization.py:79-89 of the reference)
    from oracle import cpu_reference as R

    # plain N(0,1) input like the reference's test: the literal formula rounds x*scale to bf16
    # first, so single fp8 codes may differ by one step from the fp32-multiply kernel
    x = bf16_randn((1024, 512), 13)
    q, sinv = turbo.ops.quantize_fp8(x.cuda(), torch.float8_e4m3fn, G.TENSORWISE)
    rq, _, rsinv = R.quantize_fp8_tensorwise_ref(x, torch.float8_e4m3fn)
    torch.testing.assert_close(sinv.cpu(), rsinv, rtol=1e-4, atol=1e-4)
    d = turbo.ops.dequantize_fp8(q, torch.bfloat16, G.TENSORWISE, scale_inv=sinv).cpu()
    rd = R.dequantize_fp8_ref(rq, torch.bfloat16, rsinv)
    torch.testing.assert_close(d.float(), rd.float(), rtol=1e-1, atol=1e-1)


def _tw_ex(lib, x, q, sinv, ws, status, max_probes, phantom):
    from primus_turbo import _native as N

    return lib.pt_quantize_fp8_tensorwise_ex(
        N.ptr(x), N.dtype_code(x.dtype), x.numel(), N.ptr(q), N.dtype_code(q.dtype), None, N.ptr(sinv),
        N.ptr(ws), ws.numel(), N.ptr(status), max_probes, phantom, N.stream_of(x))


def test_tensorwise_lost_grid_exchange_is_visible():
    """The bounded wait of the grid exchange is driven to its bound from the host: the launch
    waits for one slot more than it has workgroups, with a bound of a few hundred probes, so every
    wave exits normally. The failure has to show: NaN in scale_inv, the status word raised. The
    same workspace then serves a normal launch (generation-tagged slots need no clearing), and a
    launch with fewer workgroups after one with more."""
    from primus_turbo import _native as N

    lib = N.lib()
    x = bf16_randn((1024, 1024), seed=5, outlier_frac=0.001).cuda()
    oq, osinv = Q.fp8_tensorwise(to_f32_np(x), "e4m3")
    q = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    sinv = torch.zeros((), dtype=torch.float32, device="cuda")
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    ws = torch.zeros(lib.pt_quantize_fp8_tensorwise_workspace_bytes(), dtype=torch.uint8, device="cuda")

    N.check(_tw_ex(lib, x, q, sinv, ws, status, 200, 1))
    torch.cuda.synchronize()
    assert status.item() == 1, "a workgroup that gave up must raise the status word"
    assert torch.isnan(sinv).item(), "a lost exchange must poison scale_inv"
    y = turbo.ops.dequantize_fp8(q, torch.bfloat16, G.TENSORWISE, scale_inv=sinv)
    assert torch.isnan(y).all().item()

    # the same workspace, now a normal launch: bit-exact, status untouched
    status.zero_()
    N.check(_tw_ex(lib, x, q, sinv, ws, status, 0, 0))
    torch.cuda.synchronize()
    assert status.item() == 0
    assert bits_np(sinv).item() == osinv.view(np.uint32).item()
    assert np.array_equal(codes_np(q), oq)

    # fewer workgroups than the launch before (stale slots of the larger grid stay behind)
    xs = x[:3].contiguous()
    qs = torch.empty_like(xs, dtype=torch.float8_e4m3fn)
    for _ in range(3):
        N.check(_tw_ex(lib, xs, qs, sinv, ws, status, 0, 0))
    torch.cuda.synchronize()
    oq, osinv = Q.fp8_tensorwise(to_f32_np(xs), "e4m3")
    assert status.item() == 0 and bits_np(sinv).item() == osinv.view(np.uint32).item()
    assert np.array_equal(codes_np(qs), oq)
    # and more again
    N.check(_tw_ex(lib, x, q, sinv, ws, status, 0, 0))
    torch.cuda.synchronize()
    oq, osinv = Q.fp8_tensorwise(to_f32_np(x), "e4m3")
    assert status.item() == 0 and np.array_equal(codes_np(q), oq)


@pytest.mark.parametrize("dtype", [torch.float8_e4m3fn, torch.float8_e5m2])
@pytest.mark.parametrize("src", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(4096, 4096), (333, 257), (1,), (17,), (2881,), (256 * 1024 * 16 * 2 + 3,)])
def test_tensorwise_two_pass_bit_exact(shape, src, dtype):
    """The two-launch form (no exchange between workgroups) through the C ABI: same bytes and the
    same scale as the oracle, hence as the fused kernel; its workspace is deliberately dirty."""
    if (shape[0] >= 4096) and src != torch.bfloat16:
        pytest.skip("large sizes only for bf16")
    from primus_turbo import _native as N

    lib = N.lib()
    x = bf16_randn(shape, seed=21, outlier_frac=0.001, dtype=src)
    xg = x.cuda()
    q = torch.empty_like(xg, dtype=dtype)
    sinv = torch.zeros((), dtype=torch.float32, device="cuda")
    ws = torch.full((lib.pt_quantize_fp8_tensorwise_workspace_bytes(),), 0x7F, dtype=torch.uint8, device="cuda")
    for _ in range(2):
        N.check(lib.pt_quantize_fp8_tensorwise_two_pass(
            N.ptr(xg), N.dtype_code(src), xg.numel(), N.ptr(q), N.dtype_code(dtype), N.ptr(sinv), N.ptr(ws), ws.numel(),
            N.stream_of(xg)))
    torch.cuda.synchronize()
    oq, osinv = Q.fp8_tensorwise(to_f32_np(x), FMT[dtype])
    assert bits_np(sinv).item() == osinv.view(np.uint32).item()
    assert np.array_equal(codes_np(q), oq)


def test_tensorwise_two_pass_special_values_and_unaligned():
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

    prev = qi.set_tensorwise_mode("two_pass")
    try:
        x = torch.zeros(1000, dtype=torch.bfloat16)
        _check_tensorwise(x, torch.float8_e4m3fn)
        x = bf16_randn((4096,), 3)
        x[5] = float("nan")
        _check_tensorwise(x, torch.float8_e4m3fn)
        x[9] = float("inf")
        _check_tensorwise(x, torch.float8_e4m3fn)
        base = bf16_randn((4096 * 8 + 16,), 5, outlier_frac=0.01)
        for off in (1, 3, 8):
            xg = base.cuda()[off : off + 4096 * 8]
            q, sinv = turbo.ops.quantize_fp8(xg, torch.float8_e4m3fn, G.TENSORWISE)
            oq, osinv = Q.fp8_tensorwise(to_f32_np(base[off : off + 4096 * 8]), "e4m3")
            assert np.array_equal(codes_np(q), oq) and bits_np(sinv).item() == osinv.view(np.uint32).item()
    finally:
        qi.set_tensorwise_mode(prev)
    with pytest.raises(RuntimeError):
        qi.set_tensorwise_mode("three_pass")


def test_tensorwise_quantizers_on_concurrent_streams_two_pass():
    """Several streams quantizing at once: the two-launch form has no cross-workgroup wait, so
    every stream's result is exact whatever the others hold of the GPU."""
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

    prev = qi.set_tensorwise_mode("two_pass")
    try:
        xs = [bf16_randn((2048, 2048), seed=40 + i, outlier_frac=0.001) * (1 + i) for i in range(4)]
        xg = [x.cuda() for x in xs]
        streams = [torch.cuda.Stream() for _ in xs]
        torch.cuda.synchronize()
        outs = []
        for _ in range(3):
            outs = []
            for x, st in zip(xg, streams):
                with torch.cuda.stream(st):
                    outs.append(turbo.ops.quantize_fp8(x, torch.float8_e4m3fn, G.TENSORWISE))
        torch.cuda.synchronize()
        for x, (q, sinv) in zip(xs, outs):
            oq, osinv = Q.fp8_tensorwise(to_f32_np(x), "e4m3")
            assert bits_np(sinv).item() == osinv.view(np.uint32).item()
            assert np.array_equal(codes_np(q), oq)
    finally:
        qi.set_tensorwise_mode(prev)
