"""pt_quantize_fp8_tensorwise_static (the entry point that allocates nothing: its grid-exchange
words live in a static device array of the library) against pt_quantize_fp8_tensorwise (the same
kernels with a caller-provided workspace), through the C ABI, bit for bit: two calls in a row, the
second on a smaller input, then the argument checks."""

import ctypes

import numpy as np
import pytest
import torch

from helpers import bf16_randn, bits_np, codes_np

pytestmark = pytest.mark.gpu


def _call_static(lib, N, x, q, sinv, status, scale_in=None):
    return lib.pt_quantize_fp8_tensorwise_static(
        N.ptr(x), N.dtype_code(x.dtype), x.numel(), N.ptr(q), N.dtype_code(q.dtype), N.ptr(scale_in), N.ptr(sinv),
        N.ptr(status), N.stream_of(x))


def _call_workspace(lib, N, x, q, sinv, ws, scale_in=None):
    return lib.pt_quantize_fp8_tensorwise(
        N.ptr(x), N.dtype_code(x.dtype), x.numel(), N.ptr(q), N.dtype_code(q.dtype), N.ptr(scale_in), N.ptr(sinv),
        N.ptr(ws), ws.numel(), N.stream_of(x))


@pytest.mark.parametrize("qdtype", [torch.float8_e4m3fn, torch.float8_e5m2])
def test_static_entry_point_matches_workspace_entry_point(qdtype):
    from primus_turbo import _native as N

    lib = N.lib()
    ws = torch.zeros(lib.pt_quantize_fp8_tensorwise_workspace_bytes(), dtype=torch.uint8, device="cuda")
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    # a large input (every CU's workgroup takes part), then a smaller one (fewer workgroups: the
    # slots of the first call stay behind in the scratch), then an unaligned tail
    for shape, seed in (((2048, 4096), 11), ((37, 64), 12), ((1003,), 13)):
        x = bf16_randn(shape, seed=seed, outlier_frac=0.001).cuda()
        q_s = torch.empty_like(x, dtype=qdtype)
        q_w = torch.empty_like(x, dtype=qdtype)
        sinv_s = torch.zeros((), dtype=torch.float32, device="cuda")
        sinv_w = torch.zeros((), dtype=torch.float32, device="cuda")
        N.check(_call_static(lib, N, x, q_s, sinv_s, status))
        N.check(_call_workspace(lib, N, x, q_w, sinv_w, ws))
        torch.cuda.synchronize()
        assert status.item() == 0
        assert bits_np(sinv_s).item() == bits_np(sinv_w).item()
        assert np.array_equal(codes_np(q_s), codes_np(q_w)), shape
        assert np.isfinite(sinv_s.item()) and sinv_s.item() > 0

    # a given scale needs no exchange and no scratch
    x = bf16_randn((64, 128), seed=14).cuda()
    scale = torch.tensor(3.0, dtype=torch.float32, device="cuda")
    q_s = torch.empty_like(x, dtype=qdtype)
    q_w = torch.empty_like(x, dtype=qdtype)
    sinv_s = torch.zeros((), dtype=torch.float32, device="cuda")
    sinv_w = torch.zeros((), dtype=torch.float32, device="cuda")
    N.check(_call_static(lib, N, x, q_s, sinv_s, status, scale))
    N.check(_call_workspace(lib, N, x, q_w, sinv_w, ws, scale))
    torch.cuda.synchronize()
    assert np.array_equal(codes_np(q_s), codes_np(q_w)) and sinv_s.item() == sinv_w.item()


def test_static_entry_point_on_a_side_stream_and_its_limits():
    from primus_turbo import _native as N

    lib = N.lib()
    x = bf16_randn((512, 512), seed=15).cuda()
    q_ref = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    sinv_ref = torch.zeros((), dtype=torch.float32, device="cuda")
    ws = torch.zeros(lib.pt_quantize_fp8_tensorwise_workspace_bytes(), dtype=torch.uint8, device="cuda")
    N.check(_call_workspace(lib, N, x, q_ref, sinv_ref, ws))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        q = torch.empty_like(x, dtype=torch.float8_e4m3fn)
        sinv = torch.zeros((), dtype=torch.float32, device="cuda")
        for _ in range(2):
            N.check(_call_static(lib, N, x, q, sinv, None))
    side.synchronize()
    assert np.array_equal(codes_np(q), codes_np(q_ref)) and sinv.item() == sinv_ref.item()

    # sizes beyond the stated maximum are rejected before anything is launched
    too_many = ctypes.c_int64(1 << 38)
    rc = lib.pt_quantize_fp8_tensorwise_static(N.ptr(x), 0, too_many, N.ptr(q), 3, None, N.ptr(sinv), None, None)
    assert rc == N.PT_ERR_INVALID_ARGUMENT and b"MAX_NUMEL" in lib.pt_last_error()


def test_static_slot_sets_are_released_and_reused():
    """A stream handle keeps its slot set until pt_tensorwise_static_release: fill the table, see the
    next handle refused, release one, see it served, and give every set of this test back."""
    from primus_turbo import _native as N

    lib = N.lib()
    x = bf16_randn((256, 512), seed=16).cuda()
    q_ref = torch.empty_like(x, dtype=torch.float8_e4m3fn)
    sinv_ref = torch.zeros((), dtype=torch.float32, device="cuda")
    ws = torch.zeros(lib.pt_quantize_fp8_tensorwise_workspace_bytes(), dtype=torch.uint8, device="cuda")
    N.check(_call_workspace(lib, N, x, q_ref, sinv_ref, ws))
    torch.cuda.synchronize()
    streams, held, refused = [torch.cuda.Stream() for _ in range(10)], [], None
    assert len({s.cuda_stream for s in streams}) == 10
    try:
        for st in streams:
            with torch.cuda.stream(st):
                q = torch.empty_like(x, dtype=torch.float8_e4m3fn)
                sinv = torch.zeros((), dtype=torch.float32, device="cuda")
                rc = _call_static(lib, N, x, q, sinv, None)
            st.synchronize()
            if rc == N.PT_ERR_WORKSPACE:
                refused = st
                break
            N.check(rc)
            held.append(st)
            assert np.array_equal(codes_np(q), codes_np(q_ref)) and sinv.item() == sinv_ref.item()
        assert refused is not None and len(held) <= 8, "the table holds eight stream handles per device"
        # (earlier tests of the session may hold sets too: with none of this test's own, the idle
        # default stream's set is the one given back)
        victim = held[0].cuda_stream if held else torch.cuda.default_stream().cuda_stream
        assert lib.pt_tensorwise_static_release(victim) == 0
        assert lib.pt_tensorwise_static_release(victim) == 0  # holding nothing is no error
        with torch.cuda.stream(refused):
            q = torch.empty_like(x, dtype=torch.float8_e4m3fn)
            sinv = torch.zeros((), dtype=torch.float32, device="cuda")
            for _ in range(2):  # the set it inherits carries the previous owner's tags
                N.check(_call_static(lib, N, x, q, sinv, None))
        refused.synchronize()
        held = held[1:] + [refused]
        assert np.array_equal(codes_np(q), codes_np(q_ref)) and sinv.item() == sinv_ref.item()
    finally:
        torch.cuda.synchronize()
        for st in held:
            lib.pt_tensorwise_static_release(st.cuda_stream)
