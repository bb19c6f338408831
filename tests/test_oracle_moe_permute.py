"""Pins of oracle/moe_permute.py: the permuted layout built the way the reference's own test states
it (tests/pytorch/ops/test_moe_permute.py:45-75 -- expert-major, each expert's tokens in ascending
order, zero padding appended per expert), brute-force counting for tokens_per_expert /
num_dispatched, the overflow rule on a hand-sized case, and permute -> unpermute = tokens x number of
local experts. A wrong offset, a 0- instead of 1-based row or a swapped aux column fails them."""

import numpy as np
import pytest

from oracle import moe_permute as P


def _routing(T, E, K, seed, empty_rows=0):
    rng = np.random.default_rng(seed)
    flags = np.zeros((T, E), dtype=bool)
    for t in range(T - empty_rows):
        flags[t, rng.choice(E, K, replace=False)] = True
    return flags


def _layout(flags, pad):
    """(source token or -1 per permuted row)"""
    src = []
    for e in range(flags.shape[1]):
        toks = np.nonzero(flags[:, e])[0].tolist()
        src += toks
        if pad > 0:
            src += [-1] * (-len(toks) % pad)
    return np.array(src, dtype=np.int64)


@pytest.mark.parametrize("T,E,K,pad", [(64, 4, 2, 0), (100, 8, 3, 16), (37, 5, 1, 8), (256, 16, 8, 128), (50, 6, 2, 1)])
@pytest.mark.parametrize("kind", ["bool", "int32", "int64"])
def test_layout_matches_expert_major_statement(T, E, K, pad, kind):
    flags = _routing(T, E, K, seed=T + E)
    if kind == "bool":
        emap = flags
    else:
        emap = np.stack([np.nonzero(r)[0] for r in flags]).astype(kind)
        emap = emap[:, np.random.default_rng(1).permutation(K)]  # the order of the slots must not matter
    rmap, tpe, overflow, nd = P.preprocess(emap, E, pad)
    src = _layout(flags, pad)
    assert overflow == 0 and nd == T and tpe.sum() == len(src)
    per = flags.sum(0)
    assert np.array_equal(tpe, (per + pad - 1) // pad * pad if pad else per)
    tokens = np.random.default_rng(2).integers(1, 1 << 15, (T, 8)).astype(np.uint16)
    out, _, _, written = P.permute(tokens, rmap, E, len(src), pad)
    assert written.all()
    want = np.where(src[:, None] >= 0, tokens[np.maximum(src, 0)], 0)
    assert np.array_equal(out, want)


def test_probs_and_scales_follow_their_token():
    T, E, K = 40, 6, 3
    flags = _routing(T, E, K, seed=3)
    topk = np.stack([np.random.default_rng(t).permutation(np.nonzero(r)[0]) for t, r in enumerate(flags)]).astype(np.int64)
    probs_topk = np.random.default_rng(4).random((T, K)).astype(np.float32)
    rmap, _, _, _ = P.preprocess(topk, E, 4, topk_aligned_probs=True)
    src = _layout(flags, 4)
    tokens = np.arange(T * 4, dtype=np.float32).reshape(T, 4)
    sf = np.random.default_rng(5).random((T, 2)).astype(np.float32)
    out, out_sf, out_p, _ = P.permute(tokens, rmap, E, len(src), 4, scaling_factor=sf, probs=probs_topk)
    row = 0
    for e in range(E):
        for t in np.nonzero(flags[:, e])[0]:
            k = int(np.nonzero(topk[t] == e)[0][0])
            assert out_p[row] == probs_topk[t, k] and np.array_equal(out_sf[row], sf[t])
            row += 1
        while row < len(src) and src[row] == -1:
            assert out_p[row] == 0 and not out_sf[row].any()
            row += 1
    # multihot probs: the column is the expert
    probs_hot = np.random.default_rng(6).random((T, E)).astype(np.float32)
    rmap2, _, _, _ = P.preprocess(flags, E, 4)
    _, _, out_p2, _ = P.permute(tokens, rmap2, E, len(src), 4, probs=probs_hot)
    experts = np.repeat(np.arange(E), [(n + 3) // 4 * 4 for n in flags.sum(0)])
    real = src >= 0
    assert np.array_equal(out_p2[real], probs_hot[src[real], experts[real]]) and not out_p2[~real].any()


def test_overflow_rule_by_hand():
    # 3 experts with 3, 2, 1 tokens, padded to 2: rows 1-4 | 5-6 | 7-8; limit 5 keeps 4 + 1 + 0
    flags = np.zeros((4, 3), dtype=bool)
    flags[[0, 1, 2], 0] = True
    flags[[1, 3], 1] = True
    flags[2, 2] = True
    rmap, tpe, overflow, nd = P.preprocess(flags, 3, 2, num_permuted_tokens=5)
    assert overflow == 1 and nd == 4 and tpe.tolist() == [4, 1, 0]
    assert rmap[1].tolist() == [2, 5, 0, 0, 1, 0, 2]          # token 1: expert 0 row 2, expert 1 row 5
    assert rmap[3].tolist() == [0, 0, 0, 0, 0, 0, 0]          # token 3: expert 1 row 6 is beyond the limit
    assert rmap[2].tolist() == [3, 0, 0, 0, 0, 0, 1]          # token 2: expert 2 row 7 dropped
    assert rmap[4].tolist() == [-4, 0, 0, 0, 0, 0, 1]         # pad row 0: expert 0's zero row 4; expert 2's row 8 dropped
    rmap, tpe, overflow, _ = P.preprocess(flags, 3, 2)
    assert overflow == 0 and tpe.tolist() == [4, 2, 2] and rmap[4].tolist() == [-4, -8, 0, 0, 2, 0, 2]
    assert rmap[5, 6] == 0                                    # no expert needs a second zero row


def test_unpermute_round_trip_and_empty_rows():
    T, E, K = 48, 8, 3
    flags = _routing(T, E, K, seed=9, empty_rows=5)
    rmap, tpe, _, nd = P.preprocess(flags, E, 8)
    assert nd == T - 5
    tokens = np.random.default_rng(10).standard_normal((T, 16)).astype(np.float32)
    out, _, _, _ = P.permute(tokens, rmap, E, int(tpe.sum()), 8)
    back, _ = P.unpermute(out, rmap, E, T)
    assert np.allclose(back[: T - 5], tokens[: T - 5] * K, rtol=1e-6) and not back[T - 5:].any()
    # against a brute-force sum over (token, expert) pairs
    brute = np.zeros_like(tokens)
    row = 0
    for e in range(E):
        for t in np.nonzero(flags[:, e])[0]:
            brute[t] += out[row]
            row += 1
        row += -int(flags[:, e].sum()) % 8
    assert np.allclose(back, brute, rtol=1e-6)
