"""Pins for oracle/formats.py that do not reuse its formulas: torch's own CPU casts,
hand-written value tables, exhaustive midpoints and integer invariants."""

import numpy as np
import pytest
import torch

from oracle import formats as F

FP8 = [(F.E4M3, torch.float8_e4m3fn), (F.E5M2, torch.float8_e5m2)]


@pytest.mark.parametrize("fmt,tdtype", FP8)
def test_fp8_decode_table_matches_torch(fmt, tdtype):
    ref = torch.arange(256, dtype=torch.uint8).view(tdtype).float().numpy()
    assert np.array_equal(F.decode_table(fmt), ref, equal_nan=True)


@pytest.mark.parametrize("fmt,tdtype", FP8)
def test_fp8_encode_every_bf16_input(fmt, tdtype):
    x = F.bf16_bits_to_f32(np.arange(65536, dtype=np.uint16))
    x = x[np.isfinite(x)]
    xc = np.clip(x, -fmt.max_finite, fmt.max_finite)
    ref = torch.from_numpy(xc).to(tdtype).view(torch.uint8).numpy()
    assert np.array_equal(F.encode_rne(xc, fmt), ref)


@pytest.mark.parametrize("fmt,tdtype", FP8)
def test_fp8_encode_ties_and_neighbours(fmt, tdtype):
    """Every midpoint between adjacent finite codes must go to the even code; the fp32
    neighbours of the midpoint must go to their nearer code."""
    tab = F.decode_table(fmt).astype(np.float64)
    pos = np.sort(np.unique(tab[np.isfinite(tab) & (tab >= 0)]))
    pos = pos[pos <= fmt.max_finite]
    mids = ((pos[:-1] + pos[1:]) / 2).astype(np.float32)
    assert np.array_equal(mids.astype(np.float64), (pos[:-1] + pos[1:]) / 2)  # exactly representable
    below = np.nextafter(mids, np.float32(0))
    above = np.nextafter(mids, np.float32(np.inf))
    lo_codes = F.encode_rne(pos[:-1].astype(np.float32), fmt)
    hi_codes = F.encode_rne(pos[1:].astype(np.float32), fmt)
    got = F.encode_rne(mids, fmt)
    even = np.where(lo_codes % 2 == 0, lo_codes, hi_codes)
    assert np.array_equal(got, even)
    assert np.array_equal(F.encode_rne(below, fmt), lo_codes)
    assert np.array_equal(F.encode_rne(above, fmt), hi_codes)
    for arr in (mids, below, above, -mids):
        ref = torch.from_numpy(arr).to(tdtype).view(torch.uint8).numpy()
        assert np.array_equal(F.encode_rne(arr, fmt), ref)


@pytest.mark.parametrize("fmt,tdtype", FP8)
def test_fp8_encode_random_fp32(fmt, tdtype):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(200000) * np.exp2(rng.integers(-20, 10, 200000))).astype(np.float32)
    x = np.clip(x, -fmt.max_finite, fmt.max_finite)
    ref = torch.from_numpy(x).to(tdtype).view(torch.uint8).numpy()
    assert np.array_equal(F.encode_rne(x, fmt), ref)
    # float64 input takes the same path
    assert np.array_equal(F.encode_rne(x.astype(np.float64), fmt), ref)


def test_fp8_boundaries():
    assert F.encode_rne(np.float32([448.0, -448.0, 0.0]), F.E4M3).tolist() == [0x7E, 0xFE, 0x00]
    assert F.encode_rne(np.float32([57344.0, -57344.0]), F.E5M2).tolist() == [0x7B, 0xFB]
    assert F.encode_rne(np.float32([2.0**-9, 2.0**-10, 2.0**-10 * 1.0001]), F.E4M3).tolist() == [1, 0, 1]
    with pytest.raises(ValueError):
        F.encode_rne(np.float32([449.0]), F.E4M3)


def test_e2m1_table_and_midpoints():
    vals = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
    assert F.decode_table(F.E2M1).tolist() == vals + [-v for v in vals]
    for i, v in enumerate(vals):
        assert F.encode_rne(np.float32([v, -v]), F.E2M1).tolist() == [i, i + 8]
    # ties to even: 0.25->0, 0.75->1, 1.25->1, 1.75->2, 2.5->2, 3.5->4, 5->4
    ties = {0.25: 0.0, 0.75: 1.0, 1.25: 1.0, 1.75: 2.0, 2.5: 2.0, 3.5: 4.0, 5.0: 4.0}
    for t, want in ties.items():
        for s in (1.0, -1.0):
            c = F.encode_rne(np.float32([s * t]), F.E2M1)
            assert F.decode(c, F.E2M1)[0] == s * want
        lo = np.nextafter(np.float32(t), np.float32(0))
        hi = np.nextafter(np.float32(t), np.float32(10))
        i = int(np.searchsorted(vals, t))
        assert F.decode(F.encode_rne(np.float32([lo]), F.E2M1), F.E2M1)[0] == vals[i - 1]
        assert F.decode(F.encode_rne(np.float32([hi]), F.E2M1), F.E2M1)[0] == vals[i]


@pytest.mark.parametrize(
    "fmt,round_up_at,bound", [(F.E2M1, 1.75, 7.0), (F.E4M3, 1.9375, 496.0), (F.E5M2, 1.875, 61440.0)]
)
def test_e8m0_rule_over_every_bf16_amax(fmt, round_up_at, bound):
    """Brute force with python ints and math.frexp instead of the vectorised bit trick."""
    import math

    add, tgt = F.E8M0_RULE[fmt.name]
    bits = np.arange(0x0000, 0x7F80, dtype=np.uint16)  # non-negative finite bf16
    amax = F.bf16_bits_to_f32(bits)
    e = F.e8m0_exponent(amax, fmt)
    for a, ee in zip(amax[:: 7].tolist(), e[:: 7].tolist()):
        if a == 0 or a < 2.0**-126:
            continue
        m, ex = math.frexp(a)  # a = m * 2^ex, m in [0.5, 1)
        sig, unb = m * 2, ex - 1
        want = unb - tgt + (1 if sig >= round_up_at else 0)
        want = max(-127, min(128, want))
        assert ee == want, (a, ee, want)
    # scaled amax stays below the saturation sliver bound and above half the format range
    live = (amax >= 2.0**-100) & (amax < 2.0**100)
    scaled = amax[live].astype(np.float64) * np.exp2(-e[live].astype(np.float64))
    assert np.all(scaled < bound)
    assert np.all(scaled >= 2.0**tgt * (round_up_at / 2))  # never wastes more than one binade
    # specials
    assert F.e8m0_exponent(np.float32([0.0]), fmt)[0] == -127
    # inf / NaN: the exponent field 255 runs through the same integer rule (no special case)
    assert F.e8m0_exponent(np.float32([np.inf]), fmt)[0] == 255 - 127 - tgt
    assert F.e8m0_exponent(np.float32([np.nan]), fmt)[0] == 255 - 127 - tgt


def test_e8m0_to_f32():
    b = np.arange(256, dtype=np.uint8)
    v = F.e8m0_to_f32(b)
    assert v[0] == 0.0 and np.isinf(v[255])
    assert np.array_equal(v[1:255], np.exp2(np.arange(1, 255, dtype=np.float64) - 127).astype(np.float32))
    if hasattr(torch, "float8_e8m0fnu"):
        t = torch.arange(1, 255, dtype=torch.uint8).view(torch.float8_e8m0fnu).float().numpy()
        assert np.array_equal(v[1:255], t)


def test_bf16_helpers_match_torch():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(100000) * np.exp2(rng.integers(-30, 30, 100000))).astype(np.float32)
    ref = torch.from_numpy(x).to(torch.bfloat16)
    assert np.array_equal(F.f32_to_bf16_bits(x), ref.view(torch.int16).numpy().view(np.uint16))
    assert np.array_equal(F.bf16_bits_to_f32(F.f32_to_bf16_bits(x)), ref.float().numpy())
