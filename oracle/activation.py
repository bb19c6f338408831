"""CPU restatement of the gated activations (TEST INFRASTRUCTURE ONLY; only tests may import it).

Formulas of /root/reference/primus_turbo/triton/activation/swiglu_kernel.py:40-57,100-135 and
/root/reference/primus_turbo/triton/utils/gelu.py:24-49, evaluated in float64 on the exact values
of the 16-bit inputs. Floating point: parity is by tolerance (one rounding of the 16-bit output
format plus fp32 evaluation error), as in the reference's own test
(/root/reference/tests/pytorch/ops/test_activation.py:60-140, which compares against a
torch.compile'd PyTorch formula). The gate's GELU gradient here is the mathematical one; the
reference kernel multiplies it by grad_out a second time (geglu_kernel.py:126-127), which its test,
run with grad_out = 1, does not see. Pinned by central finite differences of the forward formula."""

from __future__ import annotations

import math

import numpy as np

_erf = np.vectorize(math.erf, otypes=[np.float64])


def act(g: np.ndarray, kind: str) -> np.ndarray:
    g = np.asarray(g, dtype=np.float64)
    if kind == "silu":
        return g / (1.0 + np.exp(-g))
    return 0.5 * g * (1.0 + _erf(g / math.sqrt(2.0)))


def act_grad(g: np.ndarray, kind: str) -> np.ndarray:
    g = np.asarray(g, dtype=np.float64)
    if kind == "silu":
        s = 1.0 / (1.0 + np.exp(-g))
        return s * (1.0 + g * (1.0 - s))
    return g * np.exp(-0.5 * g * g) / math.sqrt(2.0 * math.pi) + 0.5 * _erf(g / math.sqrt(2.0)) + 0.5


def glu_with_probs(x: np.ndarray, probs: np.ndarray, kind: str, row_mask=None) -> np.ndarray:
    """x [T, 2H], probs [T] -> out [T, H] (float64); masked rows are zero."""
    x = np.asarray(x, dtype=np.float64)
    H = x.shape[1] // 2
    out = act(x[:, :H], kind) * x[:, H:] * np.asarray(probs, dtype=np.float64)[:, None]
    if row_mask is not None:
        out = out * (np.asarray(row_mask) != 0)[:, None]
    return out


def glu_with_probs_grad(grad_out: np.ndarray, x: np.ndarray, probs: np.ndarray, kind: str, row_mask=None):
    """-> (grad_x [T, 2H], grad_probs [T]) in float64."""
    x, go = np.asarray(x, dtype=np.float64), np.asarray(grad_out, dtype=np.float64)
    p = np.asarray(probs, dtype=np.float64)[:, None]
    H = x.shape[1] // 2
    g, u = x[:, :H], x[:, H:]
    a, da = act(g, kind), act_grad(g, kind)
    gx = np.concatenate([go * p * u * da, go * p * a], axis=1)
    gp = (go * a * u).sum(axis=1)
    if row_mask is not None:
        m = np.asarray(row_mask) != 0
        gx, gp = gx * m[:, None], gp * m
    return gx, gp
