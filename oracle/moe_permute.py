"""CPU restatement of the MoE token permute / unpermute (TEST INFRASTRUCTURE ONLY; only tests may
import it).

Follows /root/reference/csrc/kernels/moe_permute/moe_permute.cu: routing flags from a bool map or
from topk_idx (:33-67), 1-based per-expert ranks and padded expert offsets (:150-228), the row map
with its aux columns, overflow rule and padding rows (:230-310), tokens_per_expert (:312-320), the
permute copy incl. scale factors and probs (:425-510) and the unpermute sum in fp32 (:553-620).
Integer / byte work is bit-exact; the unpermute sum is fp32 in map order, rounded once to the
16-bit format, which the kernel reproduces bit for bit.
Pinned in tests/test_oracle_moe_permute.py against the layout as the reference's own test states it
(tests/pytorch/ops/test_moe_permute.py:45-75: expert-major, tokens ascending within an expert,
zero padding per expert), against brute-force loops and the permute -> unpermute round trip."""

from __future__ import annotations

import numpy as np


def routing_flags(expert_map: np.ndarray, E: int) -> np.ndarray:
    """bool ``[T, E]`` from a bool routing map or from ``topk_idx [T, K]`` (entries outside [0, E) ignored)."""
    if expert_map.dtype == np.bool_:
        assert expert_map.shape[1] == E
        return expert_map.copy()
    T, K = expert_map.shape
    flags = np.zeros((T, E), dtype=bool)
    for k in range(K):
        col = expert_map[:, k].astype(np.int64)
        ok = (col >= 0) & (col < E)
        flags[np.nonzero(ok)[0], col[ok]] = True
    return flags


def preprocess(expert_map: np.ndarray, E: int, pad_multiple: int = 0, num_permuted_tokens: int = -1,
               topk_aligned_probs: bool = False):
    """-> (row_id_map [T + pad_multiple, 2E + 1] int32 with unused entries 0, tokens_per_expert [E]
    int64, overflow_flag, num_dispatched_tokens)."""
    flags = routing_flags(expert_map, E)
    T = flags.shape[0]
    npt = np.iinfo(np.int32).max if num_permuted_tokens <= 0 else int(num_permuted_tokens)
    real = flags.sum(axis=0).astype(np.int64)
    padded = (real + pad_multiple - 1) // pad_multiple * pad_multiple if pad_multiple > 0 else real.copy()
    prefix = np.concatenate([[0], np.cumsum(padded)[:-1]]).astype(np.int64)
    rank = np.cumsum(flags, axis=0)  # 1-based rank of a routed token within its expert
    rmap = np.zeros((T + pad_multiple, 2 * E + 1), dtype=np.int32)
    overflow = 0
    for t in range(T):
        n = 0
        for e in np.nonzero(flags[t])[0]:
            dest = int(rank[t, e] + prefix[e])
            if dest > npt:
                overflow = 1
                continue
            aux = int(e)
            if topk_aligned_probs:
                aux = int(np.nonzero(expert_map[t].astype(np.int64) == e)[0][0])
            rmap[t, n], rmap[t, E + n] = dest, aux
            n += 1
        rmap[t, 2 * E] = n
    for i in range(pad_multiple):
        n = 0
        for e in range(E):
            if i >= padded[e] - real[e]:
                continue
            off = int(real[e] + prefix[e] + i + 1)
            if off > npt:
                overflow = 1
                continue
            rmap[T + i, n], rmap[T + i, E + n] = -off, e
            n += 1
        rmap[T + i, 2 * E] = n
    over = padded + prefix - npt
    tpe = np.where(over < 0, padded, np.maximum(0, padded - over)).astype(np.int64)
    return rmap, tpe, overflow, int(flags.any(axis=1).sum())


def permute(tokens: np.ndarray, rmap: np.ndarray, E: int, rows: int, pad_multiple: int = 0, scaling_factor=None,
            probs=None, fill=None):
    """-> (permuted tokens [rows, hidden], permuted scale factors or None, permuted probs or None,
    written [rows] bool). Rows that no map entry names keep ``fill`` (0 when None)."""
    T = tokens.shape[0]
    out = np.zeros((rows,) + tokens.shape[1:], dtype=tokens.dtype) if fill is None else fill.copy()
    out_sf = None if scaling_factor is None else np.zeros((rows, scaling_factor.shape[1]), dtype=scaling_factor.dtype)
    out_p = None if probs is None else np.zeros((rows,), dtype=probs.dtype)
    written = np.zeros(rows, dtype=bool)
    for t in range(T + pad_multiple):
        for i in range(rmap[t, 2 * E]):
            d = int(rmap[t, i])
            r = d - 1 if d > 0 else -d - 1
            if d == 0 or r >= rows:
                continue
            real = d > 0 and t < T
            out[r] = tokens[t] if real else 0
            if out_sf is not None:
                out_sf[r] = scaling_factor[t] if real else 0
            if out_p is not None:
                out_p[r] = probs[t, rmap[t, E + i]] if real else 0
            written[r] = True
    return out, out_sf, out_p, written


def unpermute(permuted_f32: np.ndarray, rmap: np.ndarray, E: int, T: int, permuted_probs=None, probs_width: int = 0):
    """-> (fp32 sums [T, hidden] accumulated in map order, to be rounded once to the storage format;
    probs [T, probs_width] or None)."""
    acc = np.zeros((T, permuted_f32.shape[1]), dtype=np.float32)
    probs = None if permuted_probs is None else np.zeros((T, probs_width), dtype=permuted_probs.dtype)
    for t in range(T):
        for i in range(rmap[t, 2 * E]):
            s = int(rmap[t, i])
            if s <= 0 or s > permuted_f32.shape[0]:
                continue
            acc[t] = acc[t] + permuted_f32[s - 1].astype(np.float32)
            if probs is not None:
                probs[t, rmap[t, E + i]] = permuted_probs[s - 1]
    return acc, probs
