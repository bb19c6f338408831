"""Shared helpers for the parity tests (seeded inputs, torch <-> numpy views)."""

from __future__ import annotations

import numpy as np
import torch


def bf16_randn(shape, seed, scale=1.0, outlier_frac=0.0, outlier_mul=100.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32) * scale
    if outlier_frac > 0:
        g2 = torch.Generator().manual_seed(seed + 1)
        n = max(1, int(x.numel() * outlier_frac))
        idx = torch.randperm(x.numel(), generator=g2)[:n]
        x.view(-1)[idx] *= outlier_mul
    return x.to(dtype)


def to_f32_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().to(torch.float32).numpy()


def codes_np(t: torch.Tensor) -> np.ndarray:
    """uint8 view of an fp8 / fp4x2 / e8m0 tensor."""
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def bits_np(t: torch.Tensor) -> np.ndarray:
    """Bit pattern of a float32 / bf16 / fp16 tensor as unsigned ints."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy().view(np.uint32)
    return t.view(torch.int16).numpy().view(np.uint16)


def round_to(t_f32: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    """fp32 -> dtype with round-to-nearest-even (torch CPU cast)."""
    return torch.from_numpy(np.ascontiguousarray(t_f32)).to(dtype)


FMT = {torch.float8_e4m3fn: "e4m3", torch.float8_e5m2: "e5m2"}


def group_lens(kind, G_, total, seed):
    """Per-group row counts summing to ``total``: balanced, ragged, two non-empty groups, or
    Zipf(1.2)-skewed with two groups forced empty."""
    rng = np.random.default_rng(seed)
    if kind == "balanced":
        return np.full(G_, total // G_, dtype=np.int64)
    if kind == "ragged":
        w = 0.2 + 0.8 * rng.random(G_)
        lens = np.floor(w / w.sum() * total).astype(np.int64)
        lens[-1] += total - lens.sum()
        return lens
    if kind == "zeros":
        lens = np.zeros(G_, dtype=np.int64)
        lens[0] = total // 2
        lens[1] = total - total // 2
        return lens
    if kind == "zipf":
        w = (1.0 + np.arange(G_)) ** -1.2
        w = rng.permutation(w)
        w[rng.choice(G_, 2, replace=False)] = 0
        lens = np.floor(w / w.sum() * total).astype(np.int64)
        lens[np.argmax(lens)] += total - lens.sum()
        return lens
    raise ValueError(kind)


def gemm_gate(ref, got, what="", min_cos=0.9999, max_rel=1e-2, max_fro=1e-2, elementwise=True):
    """The GEMM gate of the parity tests: cosine similarity, error relative to the output's range,
    the Frobenius-relative error of the reference's own tests (tests/pytorch/test_utils.py:43-45) and
    an element-wise bound |err| <= 2^-7 |ref| + 2^-7 rms(ref row), under which a wrong scale on one
    row block cannot hide behind the output's range. Returns the four figures."""
    from oracle import gemm as OG

    cos, rel, fro = OG.cosine(ref, got), OG.max_rel_err(ref, got), OG.rel_fro(ref, got)
    exc = OG.elementwise_excess(ref, got) if elementwise else 0.0
    msg = f"{what}: cosine {cos:.6f}, max err / range {rel:.3e}, rel fro {fro:.3e}, element-wise excess {exc:.3f}"
    assert cos >= min_cos and rel <= max_rel and fro <= max_fro and exc <= 1.0, msg
    return {"cosine": cos, "max_rel_err": rel, "rel_fro": fro, "elementwise_excess": exc}
