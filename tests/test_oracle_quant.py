"""Pins for oracle/quantize.py: closed forms, the reference's own pure-PyTorch formula on
fp32 input, brute-force per-block loops written independently, and invariants."""

import math

import numpy as np
import pytest
import torch

from oracle import cpu_reference as R
from oracle import formats as F
from oracle import quantize as Q


def _f32(a):
    return np.asarray(a, dtype=np.float32)


def _rng_x(shape, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal(shape) * scale).astype(np.float32)
    return F.bf16_bits_to_f32(F.f32_to_bf16_bits(x))  # bf16-representable values


# ---------------------------------------------------------------- tensorwise / rowwise
def test_tensorwise_closed_forms():
    # all zero: scale = 448 / 1e-12, scale_inv = 1 / scale, all codes 0
    q, si = Q.fp8_tensorwise(np.zeros(100, np.float32), "e4m3")
    assert q.max() == 0
    s = np.float32(448.0) / np.float32(1e-12)
    assert si == np.float32(1.0) / s
    # power-of-two amax: scale is exact, element = amax -> +-448 -> 0x7E / 0xFE
    x = _f32([0.5, -4.0, 4.0, 1.0, 0.0])
    q, si = Q.fp8_tensorwise(x, "e4m3")
    assert si == np.float32(4.0 / 448.0) or si == np.float32(1.0) / np.float32(112.0)
    assert q.tolist() == [F.encode_rne(_f32([56.0]), F.E4M3)[0], 0xFE, 0x7E, F.encode_rne(_f32([112.0]), F.E4M3)[0], 0]
    # single spike: everything else collapses towards zero codes
    x = np.full(1000, 1e-3, np.float32)
    x[17] = -300.0
    q, si = Q.fp8_tensorwise(x, "e4m3")
    assert q[17] == 0xFE
    small = np.float32(1e-3) * (np.float32(448.0) / np.float32(300.0))
    assert q[0] == F.encode_rne(_f32([small]), F.E4M3)[0]
    # NaN -> +max and is ignored by the amax; inf -> scale 0
    x = _f32([1.0, np.nan, -2.0])
    q, si = Q.fp8_tensorwise(x, "e4m3")
    assert q.tolist() == [F.encode_rne(_f32([224.0]), F.E4M3)[0], 0x7E, 0xFE]
    q, si = Q.fp8_tensorwise(_f32([1.0, np.inf, -np.inf]), "e4m3")
    assert np.isinf(si) and q.tolist() == [0, 0x7E, 0x7E]
    # given scale
    q, si = Q.fp8_tensorwise(_f32([1.0, 2.0]), "e4m3", scale=_f32(2.0))
    assert si == np.float32(0.5) and q.tolist() == F.encode_rne(_f32([2.0, 4.0]), F.E4M3).tolist()


@pytest.mark.parametrize("tdtype,fmt", [(torch.float8_e4m3fn, "e4m3"), (torch.float8_e5m2, "e5m2")])
def test_tensorwise_equals_reference_formula_on_fp32(tdtype, fmt):
    """On fp32 input the reference's pure-PyTorch test formula has no extra rounding and
    must agree bit for bit (tests/pytorch/ref/quantization_ref.py:31-40 of the reference)."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(513, 257, generator=g) * 3
    x.view(-1)[::1001] *= 100
    rq, _, rsi = R.quantize_fp8_tensorwise_ref(x, tdtype)
    q, si = Q.fp8_tensorwise(x.numpy(), fmt)
    assert np.array_equal(q, rq.view(torch.uint8).numpy())
    assert si.view(np.uint32) == rsi.numpy().view(np.uint32)
    for axis in (0, 1, -1):
        # torch evaluates `scalar / tensor` as tensor.reciprocal() * scalar, i.e. with one more
        # rounding than the IEEE division of the device kernel: scales may differ by an ulp or
        # two, and only slices whose scale agrees must agree in every code.
        rq, rs, rsi = R.quantize_fp8_rowwise_ref(x, tdtype, axis)
        q, si = Q.fp8_rowwise(x.numpy(), axis, fmt)
        ulp = np.abs(si.view(np.int32).astype(np.int64) - rsi.numpy().view(np.int32).astype(np.int64))
        assert ulp.max() <= 2
        amax = np.abs(x.numpy()).max(axis=axis, keepdims=True)
        ieee_scale = (np.float32(torch.finfo(tdtype).max) / np.maximum(amax, np.float32(1e-12))).astype(np.float32)
        same_scale = ieee_scale.view(np.uint32) == rs.numpy().view(np.uint32)
        same_scale = np.broadcast_to(same_scale, q.shape)
        eq = q == rq.view(torch.uint8).numpy()
        assert np.all(eq[same_scale]) and same_scale.mean() > 0.5 and eq.mean() > 0.999
    # dequantize
    y = Q.fp8_dequant(rq.view(torch.uint8).numpy(), rsi.numpy(), fmt)
    ry = R.dequantize_fp8_ref(rq, torch.float32, rsi)
    assert np.array_equal(y.view(np.uint32), ry.numpy().view(np.uint32))


def test_rowwise_is_tensorwise_per_slice():
    x = _rng_x((5, 7, 33), 4)
    for axis in (0, 1, 2, -1, -3):
        q, si = Q.fp8_rowwise(x, axis, "e4m3")
        ax = axis % 3
        assert si.shape == tuple(1 if i == ax else s for i, s in enumerate(x.shape))
        xm, qm, sm = np.moveaxis(x, ax, -1), np.moveaxis(q, ax, -1), np.moveaxis(si, ax, -1)
        for idx in np.ndindex(xm.shape[:-1]):
            tq, tsi = Q.fp8_tensorwise(xm[idx], "e4m3")
            assert np.array_equal(tq, qm[idx]) and tsi == sm[idx][0]


# ---------------------------------------------------------------- blockwise
def _block_loop(x, r0, r1, c0, c1, qmax, fmt):
    """Independent scalar evaluation of one block (python floats + np.float32 rounding)."""
    blk = x[r0:r1, c0:c1]
    amax = np.float32(max(float(np.max(np.abs(blk))) if blk.size else 0.0, 0.0))
    scale = np.float32(qmax) / np.float32(max(amax, np.float32(1e-4)))
    v = np.clip((blk * scale).astype(np.float32), -qmax, qmax)
    return F.encode_rne(v, fmt), np.float32(1.0) / scale


@pytest.mark.parametrize("shape", [(256, 384), (130, 257), (1, 5), (300, 128)])
def test_blockwise_bruteforce(shape):
    x = _rng_x(shape, 5)
    x[0, 0] = 1000.0
    M, N = shape
    qr, sr, qc, sc = Q.fp8_blockwise_dual(x, "e4m3")
    assert sr.shape == (M, math.ceil(N / 128)) and sc.shape == (math.ceil(M / 128), N)
    for m in range(0, M, max(1, M // 7)):
        for nb in range(sr.shape[1]):
            c, s = _block_loop(x, m, m + 1, nb * 128, min(N, nb * 128 + 128), 448.0, F.E4M3)
            assert np.array_equal(c[0], qr[m, nb * 128 : nb * 128 + 128]) and s == sr[m, nb]
    for n in range(0, N, max(1, N // 7)):
        for mb in range(sc.shape[0]):
            c, s = _block_loop(x, mb * 128, min(M, mb * 128 + 128), n, n + 1, 448.0, F.E4M3)
            assert np.array_equal(c[:, 0], qc[mb * 128 : mb * 128 + 128, n]) and s == sc[mb, n]
    # weight tiles
    qw, sw = Q.fp8_blockwise_weight(x, "e4m3")
    for mb in range(sw.shape[0]):
        for nb in range(sw.shape[1]):
            c, s = _block_loop(x, mb * 128, min(M, mb * 128 + 128), nb * 128, min(N, nb * 128 + 128), 448.0, F.E4M3)
            assert np.array_equal(c, qw[mb * 128 : mb * 128 + 128, nb * 128 : nb * 128 + 128]) and s == sw[mb, nb]
    # round trip error bound: |x - deq| <= amax_block * 2^-4 (e4m3 has 3 mantissa bits)
    d = Q.fp8_blockwise_dequant(qr, sr, 1, "e4m3")
    amax = np.repeat(np.abs(np.pad(x, ((0, 0), (0, -N % 128)))).reshape(M, -1, 128).max(2), 128, axis=1)[:, :N]
    assert np.all(np.abs(d - x) <= amax * 2.0**-4 + 1e-6)


def test_blockwise_invariants():
    x = _rng_x((384, 512), 6)
    qr, sr, qc, sc = Q.fp8_blockwise_dual(x, "e5m2")
    assert (qr & 0x7F).reshape(384, 4, 128).max(2).min() == 0x7B  # every row block saturates one code
    assert (qc & 0x7F).reshape(3, 128, 512).max(1).min() == 0x7B
    a, sa = Q.fp8_blockwise(x, 1, "e5m2")
    b, sb = Q.fp8_blockwise(x, 0, "e5m2")
    assert np.array_equal(a, qr) and np.array_equal(b, qc) and np.array_equal(sa, sr) and np.array_equal(sb, sc)
    # tiny block: eps 1e-4 clamps the amax, 3-D weights are per-batch
    z = np.full((128, 128), 1e-6, np.float32)
    q, s = Q.fp8_blockwise_weight(z, "e4m3")
    assert s[0, 0] == np.float32(1.0) / (np.float32(448.0) / np.float32(1e-4))
    w = _rng_x((3, 200, 130), 7)
    q3, s3 = Q.fp8_blockwise_weight(w, "e4m3")
    for b_ in range(3):
        q2, s2 = Q.fp8_blockwise_weight(w[b_], "e4m3")
        assert np.array_equal(q3[b_], q2) and np.array_equal(s3[b_], s2)
    d = Q.fp8_blockwise_weight_dequant(q3, s3, "e4m3")
    assert d.shape == w.shape and np.max(np.abs(d - w)) < 0.3


@pytest.mark.parametrize("lens", [[128, 128], [100, 0, 30, 300], [0, 0, 5], [1] * 7, [513, 0, 127, 129]])
def test_grouped_segment_layout(lens):
    lens = np.asarray(lens, np.int64)
    M, N = int(lens.sum()), 200
    x = _rng_x((M, N), 8)
    o = Q.fp8_blockwise_segment_m_row_col(x, lens, "e4m3")
    pl, po = o["padded_lens"], o["padded_offs"]
    assert pl.tolist() == [((int(v) + 127) // 128) * 128 for v in lens]
    assert po.tolist() == [0] + np.cumsum(pl).tolist()
    Mp = M + len(lens) * 128
    assert o["col"].shape == (Mp, N) and o["col_scale"].shape == (math.ceil(Mp / 128), N)
    rq, rs = Q.fp8_blockwise(x, 1, "e4m3")
    assert np.array_equal(o["row"], rq) and np.array_equal(o["row_scale"], rs.T)
    offs = Q.group_offs(lens)
    for g, n in enumerate(lens):
        seg = o["col"][po[g] : po[g + 1]]
        assert np.all(seg[n:] == 0)  # pad rows are zero codes
        if n:
            xp = np.zeros((int(pl[g]), N), np.float32)
            xp[:n] = x[offs[g] : offs[g] + n]
            cq, cs = Q.fp8_blockwise(xp, 0, "e4m3")
            assert np.array_equal(seg, cq)
            assert np.array_equal(o["col_scale"][po[g] // 128 : po[g + 1] // 128], cs)


# ---------------------------------------------------------------- MX
@pytest.mark.parametrize("fmt,qmax", [("e4m3", 448.0), ("e5m2", 57344.0), ("e2m1", 6.0)])
def test_mx_rowwise_bruteforce(fmt, qmax):
    f = Q._fmt(fmt)
    x = _rng_x((37, 96), 9, scale=3.0)
    x[3, :32] = 0.0  # an all-zero block
    x[5, 40] = 2.0**20
    codes, sc = Q.mx_quant_rowwise(x, fmt)
    Kp = 128
    assert sc.shape == (37, Kp // 32)
    assert codes.shape == ((37, Kp // 2) if fmt == "e2m1" else (37, Kp))
    un = Q.unpack_fp4(codes) if fmt == "e2m1" else codes
    add, tgt = F.E8M0_RULE[fmt]
    for m in range(37):
        for kb in range(Kp // 32):
            blk = np.zeros(32, np.float32)
            lo, hi = kb * 32, min(96, kb * 32 + 32)
            if lo < 96:
                blk[: hi - lo] = x[m, lo:hi]
            amax = float(np.max(np.abs(blk)))
            if amax == 0:
                e = -127
            else:
                mm, ex = math.frexp(amax)
                bits = int(np.float32(amax).view(np.uint32))
                e = (((bits + add) >> 23) & 0x1FF) - 127 - tgt
                e = max(-127, min(128, e))
                assert e in (ex - 1 - tgt, ex - tgt)
            assert sc[m, kb] == e + 127
            want = F.encode_rne(np.clip(blk.astype(np.float64) * 2.0 ** (-e), -qmax, qmax), f)
            assert np.array_equal(un[m, kb * 32 : kb * 32 + 32], want)
    assert sc[3, 0] == 0 and np.all(un[3, :32] == 0)
    assert np.all(sc[:, 3] == 0) and np.all(un[:, 96:] == 0)  # K padding
    # round trip: |x - deq| <= 2^e * (half a step at the top binade)
    d = Q.mx_dequant(codes, sc, fmt)[:, :96]
    # e4m3: the block maximum may sit in the saturating sliver [448, 496) -> up to 9.7 % off
    step = {"e4m3": 0.1, "e5m2": 2.0**-3, "e2m1": 2.0**-2}[fmt]
    blk_amax = np.repeat(np.abs(np.pad(x, ((0, 0), (0, 32)))).reshape(37, 4, 32).max(2), 32, axis=1)[:, :96]
    assert np.all(np.abs(d - x) <= blk_amax * step * 1.0001 + 1e-30)


def test_mx_colwise_and_2d():
    x = _rng_x((96, 64), 10)
    c, s = Q.mx_quant_colwise(x, "e4m3")
    c2, s2 = Q.mx_quant_rowwise(np.ascontiguousarray(x.T), "e4m3")
    assert c.shape == (64, 128) and s.shape == (64, 4)
    assert np.array_equal(c, c2) and np.array_equal(s, s2)
    # 2-D blocks: one exponent per 32x32 tile, equal to the 1-D rule on the tile amax
    c, s = Q.mx_quant_rowwise(x, "e2m1", use_2d_block=True)
    for tm in range(3):
        for tk in range(2):
            tile = x[tm * 32 : tm * 32 + 32, tk * 32 : tk * 32 + 32]
            e = F.e8m0_exponent(np.float32(np.abs(tile).max()), F.E2M1)
            assert np.all(s[tm * 32 : tm * 32 + 32, tk] == e + 127)
    assert np.all(s[:, 2:] == 0)


def test_fp4_packing_order():
    codes = np.arange(16, dtype=np.uint8)[None, :]
    p = Q._pack_fp4(codes)
    assert p.tolist() == [[0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]]  # even element in the low nibble
    assert np.array_equal(Q.unpack_fp4(p), codes)


@pytest.mark.parametrize("lens", [[100, 0, 37, 163], [128, 128], [1], [0, 5, 0, 250, 31]])
@pytest.mark.parametrize("fmt,ra,ca", [("e4m3", 32, 128), ("e5m2", 32, 128), ("e2m1", 32, 128), ("e2m1", 1, 256)])
def test_mx_grouped_layout(lens, fmt, ra, ca):
    """Grouped MX quantizer: group starts on multiples of 32 (rows) / 128 (transposed columns) --
    grouped MXFP4: rows in place, columns on multiples of 256 --, every group's slice equals the
    dense quantizer of that group's rows, pads are zero codes with scale byte 0, and the round
    trip through the de-quantizer matches the dense round trip."""
    lens = np.array(lens, dtype=np.int64)
    M, N = int(lens.sum()), 160
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((M, N)) * np.exp(rng.standard_normal((M, 1)))).astype(np.float32)
    o = Q.mx_grouped_quant(x, lens, fmt, row_align=ra, col_align=ca)
    cpb = 2 if fmt == "e2m1" else 1
    assert np.all(o["row_offs"] % ra == 0) and np.all(o["col_offs"] % ca == 0)
    assert np.array_equal(o["row_lens"], (lens + ra - 1) // ra * ra) and np.array_equal(o["col_lens"], (lens + ca - 1) // ca * ca)
    if ra == 1:
        assert np.array_equal(o["row_offs"], np.concatenate([[0], np.cumsum(lens)]))
    assert o["row"].shape == (o["row_offs"][-1], 256 // cpb) and o["col"].shape == (N, o["col_offs"][-1] // cpb)
    starts = np.concatenate([[0], np.cumsum(lens)])
    for g, n in enumerate(lens):
        r0, c0, c1 = o["row_offs"][g], o["col_offs"][g], o["col_offs"][g + 1]
        seg = x[starts[g] : starts[g] + n]
        if n:
            q, s = Q.mx_quant_rowwise(seg, fmt)
            assert np.array_equal(o["row"][r0 : r0 + n], q) and np.array_equal(o["row_scale"][r0 : r0 + n], s)
            deq = Q.mx_dequant(o["col"][:, c0 // cpb : c1 // cpb], o["col_scale"][:, c0 // 32 : c1 // 32], fmt)
            qc, sc = Q.mx_quant_colwise(seg, fmt)
            assert np.array_equal(deq[:, :n], Q.mx_dequant(qc, sc, fmt)[:, :n])
            assert not deq[:, n:].any()
        pad = slice(r0 + n, o["row_offs"][g + 1])
        assert not o["row"][pad].any() and not o["row_scale"][pad].any()
        # scale bytes of blocks that lie entirely in the column padding are zero
        assert not o["col_scale"][:, (c0 + n + 31) // 32 : c1 // 32].any()


def test_mx_grouped_2d_blocks():
    """32 x 32 blocks in the grouped quantizer are counted from each group's first row: a group's
    slice equals the dense 2-D quantizer of that group's rows, its pad rows are zero codes that
    carry the exponent of their block, and every block de-quantizes with one exponent."""
    lens = np.array([40, 0, 64, 7], dtype=np.int64)
    M, N = int(lens.sum()), 96
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((M, N)) * np.exp(rng.standard_normal((M, 1)))).astype(np.float32)
    o = Q.mx_grouped_quant(x, lens, "e4m3", row_2d=True, col_2d=True)
    starts = np.concatenate([[0], np.cumsum(lens)])
    for g, n in enumerate(lens):
        if n == 0:
            continue
        r0, r1, c0 = o["row_offs"][g], o["row_offs"][g + 1], o["col_offs"][g]
        seg = x[starts[g] : starts[g] + n]
        q, s = Q.mx_quant_rowwise(seg, "e4m3", True)
        assert np.array_equal(o["row"][r0 : r0 + n], q) and np.array_equal(o["row_scale"][r0 : r0 + n], s)
        assert not o["row"][r0 + n : r1].any()
        blk = o["row_scale"][r0:r1].reshape((r1 - r0) // 32, 32, -1)
        assert np.all(blk == blk[:, :1]), "one exponent per 32 x 32 block, pad rows included"
        qc, sc = Q.mx_quant_colwise(seg, "e4m3", True)
        assert np.array_equal(o["col"][:, c0 : c0 + qc.shape[1]], qc) and np.array_equal(o["col_scale"][:, c0 // 32 : c0 // 32 + sc.shape[1]], sc)
        # the exponent of a block is that of its abs-max: the row and the column direction agree on it
        assert np.array_equal(s[::32, : N // 32], sc[::32, : -(-n // 32)].T[: -(-n // 32)][:, : N // 32])


def test_hadamard16_is_the_orthonormal_sylvester_matrix():
    """``hadamard16`` against scipy's Sylvester construction where fp32 arithmetic is exact (small
    integers), its involution, norm preservation, and what the recipe relies on: the transform
    cancels in a product of two operands that both carry it along the reduction axis."""
    import scipy.linalg

    H = scipy.linalg.hadamard(16).astype(np.float64)
    rng = np.random.default_rng(11)
    x = rng.integers(-64, 65, size=(7, 48)).astype(np.float32)
    y = Q.hadamard16(x)
    want = np.concatenate([x[:, 16 * i : 16 * i + 16].astype(np.float64) @ H.T / 4 for i in range(3)], axis=1)
    assert np.array_equal(y.astype(np.float64), want)
    assert np.array_equal(Q.hadamard16(y), x)
    e = np.zeros((16, 16), np.float32)
    np.fill_diagonal(e, 4.0)
    assert np.array_equal(Q.hadamard16(e), H.astype(np.float32))  # rows of 4 I -> rows of H (symmetric)
    g = rng.standard_normal((64, 5)).astype(np.float32)
    a = rng.standard_normal((64, 3)).astype(np.float32)
    gt, at = Q.hadamard16(g.T.copy()), Q.hadamard16(a.T.copy())
    assert np.allclose(gt @ at.T, g.T @ a, rtol=1e-5, atol=1e-5)
    assert np.allclose(np.linalg.norm(gt, axis=1), np.linalg.norm(g.T, axis=1), rtol=1e-6)


@pytest.mark.parametrize("shape", [(64, 64), (40, 96), (33, 160)])
def test_mxfp4_hadamard_quantizer(shape):
    """With ``use_rht`` the quantizer is the plain MXFP4 quantizer of the transformed, zero-padded
    tensor; an outlier is spread over its 16 neighbours (smaller block maximum, better SNR of the
    de-quantized inverse transform on spiky data)."""
    rng = np.random.default_rng(12)
    x = rng.standard_normal(shape).astype(np.float32)
    x[rng.integers(0, shape[0], 6), rng.integers(0, shape[1], 6)] *= 40
    x = F.bf16_bits_to_f32(F.f32_to_bf16_bits(x))
    q, s = Q.mx_quant_rowwise(x, "e2m1", use_rht=True)
    Kp = -(-shape[1] // 128) * 128
    xp = np.zeros((shape[0], Kp), np.float32)
    xp[:, : shape[1]] = x
    q2, s2 = Q.mx_quant_rowwise(Q.hadamard16(xp), "e2m1")
    assert np.array_equal(q, q2) and np.array_equal(s, s2)
    qc, sc = Q.mx_quant_colwise(x, "e2m1", use_rht=True)
    q3, s3 = Q.mx_quant_rowwise(np.ascontiguousarray(x.T), "e2m1", use_rht=True)
    assert np.array_equal(qc, q3) and np.array_equal(sc, s3)
    back = Q.hadamard16(Q.mx_dequant(q, s, "e2m1"))[:, : shape[1]]
    plain = Q.mx_dequant(*Q.mx_quant_rowwise(x, "e2m1"), "e2m1")[:, : shape[1]]
    err = lambda y: float(np.linalg.norm(y - x) / np.linalg.norm(x))  # noqa: E731
    assert err(back) < 0.25 and err(plain) < 0.25
