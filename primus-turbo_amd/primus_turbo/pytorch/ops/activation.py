"""``swiglu_with_probs`` / ``geglu_with_probs``: the gated activation between the two grouped GEMMs
of an MoE expert MLP, with the router probability of each token folded in, and autograd
(reference: primus_turbo/pytorch/ops/activation.py:21-83)."""

from __future__ import annotations

from typing import Optional

import torch

from primus_turbo.pytorch.kernels.activation.glu_impl import ACT_GELU, ACT_SILU, glu_bwd_with_probs, glu_fwd_with_probs

__all__ = ["swiglu_with_probs", "geglu_with_probs"]

_ACTS = {"silu": ACT_SILU, "gelu": ACT_GELU}


class GLUWithProbs(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x: torch.Tensor, probs: torch.Tensor, row_mask: Optional[torch.Tensor], act_type: str):
        assert act_type in _ACTS, f"Unsupported act_type: {act_type}. Supported types: {list(_ACTS)}"
        x_shape, probs_shape = x.size(), probs.size()
        x2, p1 = x.reshape(-1, x.size(-1)), probs.reshape(-1)
        assert x2.size(0) == p1.size(0), "first dimension of x and probs must be the same"
        assert probs.dtype == torch.float32, "probs must be float32"
        if row_mask is not None:
            assert row_mask.is_cuda, "row_mask must be a CUDA tensor"
            assert row_mask.ndim == 1 and x2.size(0) == row_mask.size(0), "row_mask must be 1D with one entry per token"
            assert row_mask.dtype == torch.int64, "The dtype of row_mask must be torch.int64."
        out = glu_fwd_with_probs(x2, p1, row_mask, _ACTS[act_type])
        ctx.save_for_backward(x2, p1, row_mask)
        ctx.meta = (_ACTS[act_type], x_shape, probs_shape)
        return out

    @staticmethod
    def backward(ctx, grad_output: torch.Tensor):
        assert grad_output.ndim == 2
        x2, p1, row_mask = ctx.saved_tensors
        act, x_shape, probs_shape = ctx.meta
        grad_x, grad_probs = glu_bwd_with_probs(grad_output, x2, p1, row_mask, act)
        return grad_x.view(x_shape), grad_probs.view(probs_shape), None, None


def swiglu_with_probs(x: torch.Tensor, probs: torch.Tensor, row_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(x[..., :H]) * x[..., H:] * probs[..., None]`` over the flattened tokens -> ``[tokens, H]``."""
    return GLUWithProbs.apply(x, probs, row_mask, "silu")


def geglu_with_probs(x: torch.Tensor, probs: torch.Tensor, row_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``gelu(x[..., :H]) * x[..., H:] * probs[..., None]`` (exact erf GELU) -> ``[tokens, H]``."""
    return GLUWithProbs.apply(x, probs, row_mask, "gelu")
