"""GPU parity of ``moe_permute`` / ``moe_unpermute`` and their dispatcher ops against
oracle/moe_permute.py. Cases follow the reference's tests/pytorch/ops/test_moe_permute.py (routing
map and topk_idx int32 / int64 forms, top-k 1 ... 8, 16 experts, per-expert padding, probs in both
layouts, FP8 tokens with scale factors, a capped output with the overflow flag) plus ragged token
counts, tokens routed nowhere and out-of-range expert ids. The row map, counts, copied bytes and
probs are compared bit for bit; the unpermute sum (fp32 in map order, one rounding) as well."""

import numpy as np
import pytest
import torch

from oracle import moe_permute as P

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _turbo(native_lib):
    global turbo, ext
    import primus_turbo.pytorch as turbo

    ext = torch.ops.primus_turbo_cpp_extension


def _routing(T, E, K, seed, empty_rows=0):
    rng = np.random.default_rng(seed)
    flags = np.zeros((T, E), dtype=bool)
    for t in range(T - empty_rows):
        flags[t, rng.choice(E, K, replace=False)] = True
    return flags


def _topk(flags, K, dtype, seed, fill_empty=-1):
    rng = np.random.default_rng(seed)
    out = np.full((flags.shape[0], K), fill_empty, dtype=dtype)
    for t, r in enumerate(flags):
        e = np.nonzero(r)[0]
        if len(e):
            out[t] = rng.permutation(e)
    return out


def _bits(t):
    return t.detach().contiguous().cpu().view(torch.uint8 if t.element_size() == 1 else torch.int16 if t.element_size() == 2
                                              else torch.int32).numpy()


@pytest.mark.parametrize("T,E,K", [(4096, 16, 1), (4096, 16, 8), (1000, 64, 4), (37, 4, 2), (257, 240, 3), (70000, 8, 2)])
@pytest.mark.parametrize("kind", ["bool", "int32", "int64"])
@pytest.mark.parametrize("pad", [0, 16, 128])
def test_preprocessing_matches_oracle(T, E, K, kind, pad):
    empty = min(5, T // 4)
    flags = _routing(T, E, K, seed=T + E + K, empty_rows=empty)
    aligned = kind != "bool" and (T + pad) % 2 == 0
    emap = flags if kind == "bool" else _topk(flags, K, kind, 3, fill_empty=E + 7 if kind == "int32" else -1)
    got = ext.permute_preprocessing(torch.from_numpy(emap).cuda(), E, K, pad, -1, K if aligned else 0)
    rmap, tpe, overflow, nd = P.preprocess(emap, E, pad, topk_aligned_probs=aligned)
    assert np.array_equal(got[0].cpu().numpy(), rmap)
    assert np.array_equal(got[1].cpu().numpy(), tpe) and got[1].dtype == torch.int64
    assert int(got[2].item()) == overflow == 0 and int(got[3].item()) == nd == T - empty


@pytest.mark.parametrize("limit", [1, 1500, 4096, 8191, 8192, 9000])
def test_preprocessing_overflow(limit):
    T, E, K, pad = 2048, 16, 4, 32
    flags = _routing(T, E, K, seed=limit)
    got = ext.permute_preprocessing(torch.from_numpy(flags).cuda(), E, K, pad, limit, 0)
    rmap, tpe, overflow, nd = P.preprocess(flags, E, pad, num_permuted_tokens=limit)
    assert np.array_equal(got[0].cpu().numpy(), rmap) and np.array_equal(got[1].cpu().numpy(), tpe)
    assert int(got[2].item()) == overflow and int(got[3].item()) == nd
    assert overflow == int(limit < int(((flags.sum(0) + pad - 1) // pad * pad).sum()))


@pytest.mark.parametrize("T,E,K,H", [(4096, 16, 2, 4096), (1000, 8, 4, 1024), (37, 4, 1, 64), (513, 32, 8, 7168)])
@pytest.mark.parametrize("pad", [0, 16])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["none", "routing_map", "topk"])
def test_permute_unpermute_match_oracle(T, E, K, H, pad, dtype, layout):
    flags = _routing(T, E, K, seed=T + H, empty_rows=2)
    topk = _topk(flags, K, np.int64, 5)
    emap = flags if layout == "routing_map" else topk
    g = torch.Generator().manual_seed(11)
    tokens = torch.randn(T, H, generator=g).to(dtype)
    probs = None
    if layout == "routing_map":
        probs = torch.rand(T, E, generator=g)
    elif layout == "topk":
        probs = torch.rand(T, K, generator=g)
    kw = dict(num_local_experts=E, num_topk=K, pad_multiple=pad)
    if layout != "none":
        kw.update(probs=probs.cuda(), probs_layout=layout)
    elif emap.dtype != bool:
        kw.update(probs_layout="routing_map")
    out, rmap_d, tpe_d, flag_d, nd_d, out_sf, out_p = turbo.ops.moe_permute(tokens.cuda(), torch.from_numpy(emap).cuda(), **kw)
    rmap, tpe, overflow, nd = P.preprocess(emap, E, pad, topk_aligned_probs=layout == "topk")
    assert np.array_equal(rmap_d.cpu().numpy(), rmap) and np.array_equal(tpe_d.cpu().numpy(), tpe)
    rows = int(tpe.sum())
    assert out.shape == (rows, H) and out_sf is None and (out_p is None) == (probs is None)
    want, _, want_p, written = P.permute(_bits(tokens), rmap, E, rows, pad, probs=None if probs is None else probs.numpy())
    assert written.all() and np.array_equal(_bits(out), want)
    if probs is not None:
        assert np.array_equal(out_p.cpu().numpy(), want_p)
    # back: every expert "output" is its input times (1 + row / 4096) so that the sum's order shows
    y = (out.float() * (1 + torch.arange(rows, device="cuda").float()[:, None] / 4096)).to(dtype)
    stride = K if layout == "topk" else 0
    back, back_p = turbo.ops.moe_unpermute(y, rmap_d, nd_d, restore_shape=tokens.shape, num_local_experts=E,
                                           permuted_probs=out_p, probs_topk_stride=stride, pad_multiple=pad)
    acc, probs_back = P.unpermute(y.float().cpu().numpy(), rmap, E, T,
                                  None if out_p is None else out_p.cpu().numpy(), stride if stride else E)
    assert np.array_equal(_bits(back), _bits(torch.from_numpy(acc).to(dtype)))
    if probs is not None:
        assert np.array_equal(back_p.cpu().numpy(), probs_back)
        hot = torch.from_numpy(flags)
        if layout == "routing_map":
            assert torch.equal(back_p.cpu(), torch.where(hot, probs, torch.zeros(())))


def test_permute_fp8_tokens_with_scale_factors():
    T, E, K, H, S, pad = 777, 8, 2, 2048, 16, 8
    flags = _routing(T, E, K, seed=21)
    tok = torch.from_numpy(np.random.default_rng(22).integers(0, 256, (T, H), dtype=np.uint8)).view(torch.float8_e4m3fn)
    sf = torch.rand(T, S, generator=torch.Generator().manual_seed(23))
    out, rmap_d, tpe_d, _, _, out_sf, out_p = turbo.ops.moe_permute(
        tok.cuda(), torch.from_numpy(flags).cuda(), num_local_experts=E, num_topk=K, pad_multiple=pad,
        scaling_factor=sf.cuda(), scales_per_token=S, use_fp8=True, probs_layout="routing_map")
    rmap, tpe, _, _ = P.preprocess(flags, E, pad)
    want, want_sf, _, written = P.permute(_bits(tok), rmap, E, int(tpe.sum()), pad, scaling_factor=sf.numpy())
    assert written.all() and out.dtype == torch.float8_e4m3fn and out_p is None
    assert np.array_equal(_bits(out), want) and np.array_equal(out_sf.cpu().numpy(), want_sf)


def test_capped_output_drops_rows_and_flags_overflow():
    T, E, K, H, pad = 512, 8, 2, 256, 16
    flags = _routing(T, E, K, seed=31)
    tokens = torch.randn(T, H, generator=torch.Generator().manual_seed(32)).to(torch.bfloat16)
    limit = 700  # < 1024 routed rows
    out, rmap_d, tpe_d, flag_d, _, _, _ = turbo.ops.moe_permute(
        tokens.cuda(), torch.from_numpy(flags).cuda(), num_local_experts=E, num_topk=K, pad_multiple=pad,
        num_permuted_tokens=limit, probs_layout="routing_map")
    rmap, tpe, overflow, _ = P.preprocess(flags, E, pad, num_permuted_tokens=limit)
    assert out.shape[0] == limit and int(flag_d.item()) == overflow == 1 and np.array_equal(tpe_d.cpu().numpy(), tpe)
    want, _, _, written = P.permute(_bits(tokens), rmap, E, limit, pad)
    assert written.all() and np.array_equal(_bits(out), want)


@pytest.mark.parametrize("layout", ["routing_map", "topk"])
def test_autograd_of_both_directions(layout):
    T, E, K, H, pad = 300, 8, 3, 512, 8
    flags = _routing(T, E, K, seed=41, empty_rows=3)
    topk = _topk(flags, K, np.int32, 42)
    emap = torch.from_numpy(flags if layout == "routing_map" else topk).cuda()
    g = torch.Generator().manual_seed(43)
    tokens = torch.randn(T, H, generator=g).to(torch.bfloat16).cuda().requires_grad_(True)
    probs = torch.rand(T, E if layout == "routing_map" else K, generator=g).cuda().requires_grad_(True)
    out, rmap_d, tpe_d, _, nd_d, _, out_p = turbo.ops.moe_permute(
        tokens, emap, num_local_experts=E, num_topk=K, pad_multiple=pad, probs=probs, probs_layout=layout)
    rows = out.shape[0]
    w = torch.randn(rows, H, generator=g).to(torch.bfloat16).cuda()
    wp = torch.rand(rows, generator=g).cuda()
    (out.float() * w.float()).sum().backward(retain_graph=True)
    (out_p * wp).sum().backward()
    rmap = rmap_d.cpu().numpy()
    stride = K if layout == "topk" else 0
    acc, gp = P.unpermute(w.float().cpu().numpy(), rmap, E, T, wp.cpu().numpy(), stride if stride else E)
    assert np.array_equal(_bits(tokens.grad), _bits(torch.from_numpy(acc).to(torch.bfloat16)))
    assert np.array_equal(probs.grad.cpu().numpy(), gp)
    # unpermute forward, permute backward
    y = out.detach().clone().requires_grad_(True)
    yp = out_p.detach().clone().requires_grad_(True)
    back, back_p = turbo.ops.moe_unpermute(y, rmap_d, nd_d, restore_shape=tokens.shape, num_local_experts=E,
                                           permuted_probs=yp, probs_topk_stride=stride, pad_multiple=pad)
    gt = torch.randn(T, H, generator=g).to(torch.bfloat16).cuda()
    gpb = torch.rand(back_p.shape, generator=g).cuda()
    torch.autograd.backward([back, back_p], [gt, gpb])
    want, _, want_p, _ = P.permute(_bits(gt), rmap, E, rows, pad, probs=gpb.cpu().numpy())
    assert np.array_equal(_bits(y.grad), want) and np.array_equal(yp.grad.cpu().numpy(), want_p)


def test_no_tokens_and_argument_checks():
    E = 4
    out = turbo.ops.moe_permute(torch.empty(0, 128, dtype=torch.bfloat16, device="cuda"),
                                torch.empty(0, E, dtype=torch.bool, device="cuda"), num_local_experts=E, num_topk=2,
                                pad_multiple=8, probs_layout="routing_map")
    assert out[0].shape == (0, 128) and out[1].shape == (8, 2 * E + 1) and int(out[2].sum()) == 0
    with pytest.raises(ValueError, match="probs_layout"):
        turbo.ops.moe_permute(torch.empty(4, 128, device="cuda"), torch.zeros(4, E, dtype=torch.bool, device="cuda"),
                              num_local_experts=E, probs_layout="dense")
    with pytest.raises(RuntimeError, match="second dimension must equal num_local_experts"):
        ext.permute_preprocessing(torch.zeros(4, E + 1, dtype=torch.bool, device="cuda"), E, 2, 0, -1, 0)
    with pytest.raises(RuntimeError, match="requires the topk_idx"):
        ext.permute_preprocessing(torch.zeros(4, E, dtype=torch.bool, device="cuda"), E, 2, 0, -1, 2)
    with pytest.raises(RuntimeError, match="num_local_experts must be in"):
        ext.permute_preprocessing(torch.zeros(4, 300, dtype=torch.bool, device="cuda"), 300, 2, 0, -1, 0)
    with pytest.raises(RuntimeError, match="bool or int or int64"):
        ext.permute_preprocessing(torch.zeros(4, E, dtype=torch.float32, device="cuda"), E, 2, 0, -1, 0)


@pytest.mark.parametrize("layout", ["routing_map", "topk"])
def test_half_precision_probs(layout):
    """Probabilities are moved as raw 2-byte values too (bf16 routers)."""
    T, E, K, H, pad = 333, 8, 2, 256, 4
    flags = _routing(T, E, K, seed=51)
    topk = _topk(flags, K, np.int64, 52)
    emap = flags if layout == "routing_map" else topk
    g = torch.Generator().manual_seed(53)
    tokens = torch.randn(T, H, generator=g).to(torch.bfloat16)
    probs = torch.rand(T, E if layout == "routing_map" else K, generator=g).to(torch.bfloat16)
    out, rmap_d, tpe_d, _, nd_d, _, out_p = turbo.ops.moe_permute(
        tokens.cuda(), torch.from_numpy(emap).cuda(), num_local_experts=E, num_topk=K, pad_multiple=pad,
        probs=probs.cuda(), probs_layout=layout)
    rmap, tpe, _, _ = P.preprocess(emap, E, pad, topk_aligned_probs=layout == "topk")
    _, _, want_p, _ = P.permute(_bits(tokens), rmap, E, int(tpe.sum()), pad, probs=_bits(probs))
    assert out_p.dtype == torch.bfloat16 and np.array_equal(_bits(out_p), want_p)
    stride = K if layout == "topk" else 0
    _, back_p = turbo.ops.moe_unpermute(out, rmap_d, nd_d, restore_shape=tokens.shape, num_local_experts=E,
                                        permuted_probs=out_p, probs_topk_stride=stride, pad_multiple=pad)
    _, want_back = P.unpermute(np.zeros((int(tpe.sum()), 1), np.float32), rmap, E, T, want_p, stride if stride else E)
    assert back_p.dtype == torch.bfloat16 and np.array_equal(_bits(back_p), want_back)
