"""Gated activations with the router probability folded in, forward and backward, on the gfx950
kernels (reference: primus_turbo/pytorch/kernels/activation/swiglu_impl.py:20-117 and
geglu_impl.py, which launch the Triton kernels of primus_turbo/triton/activation/)."""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from primus_turbo import _native as N

ACT_SILU, ACT_GELU = 0, 1


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _common(x, probs, row_mask):
    N.require_cuda(x, probs, row_mask)
    _check(x.dim() == 2 and x.shape[1] % 2 == 0, "x must be [tokens, 2 * hidden]")
    _check(x.dtype in (torch.bfloat16, torch.float16), "x must be bfloat16 or float16")
    _check(probs.dtype == torch.float32 and probs.numel() == x.shape[0], "probs must be float32 [tokens]")
    if row_mask is not None:
        _check(row_mask.dtype == torch.int64 and row_mask.dim() == 1 and row_mask.numel() == x.shape[0],
               "row_mask must be int64 [tokens]")
        row_mask = row_mask.contiguous()
    return x.contiguous(), probs.contiguous().view(-1), row_mask


@torch.library.custom_op("primus_turbo::glu_fwd_with_probs", mutates_args=())
def glu_fwd_with_probs(x: torch.Tensor, probs: torch.Tensor, row_mask: Optional[torch.Tensor], act: int) -> torch.Tensor:
    """``out[t] = act(x[t, :H]) * x[t, H:] * probs[t]``; rows with ``row_mask == 0`` come out as zeros."""
    x, probs, row_mask = _common(x, probs, row_mask)
    T, H = x.shape[0], x.shape[1] // 2
    out = torch.empty((T, H), dtype=x.dtype, device=x.device)
    N.check(N.lib().pt_glu_with_probs_fwd(N.ptr(x), N.dtype_code(x.dtype), N.ptr(probs), N.ptr(row_mask), N.ptr(out), T, H,
                                          act, N.stream_of(x)))
    return out


@glu_fwd_with_probs.register_fake
def _glu_fwd_with_probs_fake(x, probs, row_mask, act):
    return torch.empty((x.shape[0], x.shape[1] // 2), dtype=x.dtype, device=x.device)


@torch.library.custom_op("primus_turbo::glu_bwd_with_probs", mutates_args=())
def glu_bwd_with_probs(grad_out: torch.Tensor, x: torch.Tensor, probs: torch.Tensor, row_mask: Optional[torch.Tensor],
                       act: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """-> ``(grad_x [tokens, 2 H], grad_probs`` shaped like ``probs)``."""
    shape = probs.shape
    x, probs, row_mask = _common(x, probs, row_mask)
    T, H = x.shape[0], x.shape[1] // 2
    _check(tuple(grad_out.shape) == (T, H) and grad_out.dtype == x.dtype, "grad_out must be [tokens, hidden] in x's dtype")
    grad_out = grad_out.contiguous()
    grad_x = torch.empty_like(x)
    grad_probs = torch.empty(T, dtype=torch.float32, device=x.device)
    N.check(N.lib().pt_glu_with_probs_bwd(N.ptr(grad_out), N.ptr(x), N.dtype_code(x.dtype), N.ptr(probs), N.ptr(row_mask),
                                          N.ptr(grad_x), N.ptr(grad_probs), T, H, act, N.stream_of(x)))
    return grad_x, grad_probs.view(shape)


@glu_bwd_with_probs.register_fake
def _glu_bwd_with_probs_fake(grad_out, x, probs, row_mask, act):
    return torch.empty(x.shape, dtype=x.dtype, device=x.device), torch.empty(probs.shape, dtype=torch.float32,
                                                                              device=x.device)


def swiglu_fwd_with_probs(x, probs, row_mask=None):
    return glu_fwd_with_probs(x, probs, row_mask, ACT_SILU)


def swiglu_bwd_with_probs(grad_out, x, probs, row_mask=None):
    return glu_bwd_with_probs(grad_out, x, probs, row_mask, ACT_SILU)


def geglu_fwd_with_probs(x, probs, row_mask=None):
    return glu_fwd_with_probs(x, probs, row_mask, ACT_GELU)


def geglu_bwd_with_probs(grad_out, x, probs, row_mask=None):
    return glu_bwd_with_probs(grad_out, x, probs, row_mask, ACT_GELU)
