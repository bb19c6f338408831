"""Small helpers shared by the GEMM ops (reference: primus_turbo/pytorch/ops/utils.py:20-89)."""

from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from primus_turbo.pytorch.core.low_precision import Format, float8_e4m3, float8_e5m2


def _get_fp8_dtype(format: Format, is_fwd_stage: bool) -> torch.dtype:
    """E4M3 / E5M2 as configured; HYBRID = E4M3 for forward operands, E5M2 for gradients."""
    if format == Format.E4M3:
        return float8_e4m3
    if format == Format.E5M2:
        return float8_e5m2
    if format == Format.HYBRID:
        return float8_e4m3 if is_fwd_stage else float8_e5m2
    raise ValueError(f"Unsupported FP8 format: {format}")


def _ensure_contiguous_grad_out(grad_out: torch.Tensor) -> torch.Tensor:
    return grad_out if grad_out.is_contiguous() else grad_out.contiguous()


def _setup_fused_grad_accum(b, pattern: Optional[str]) -> Tuple[bool, Optional[torch.Tensor]]:
    """Resolve the buffer the fused wgrad accumulates into. Must run in ``forward`` while the
    weight object (which carries ``main_grad``) is in hand; flags the weight so the training
    framework skips its own accumulation."""
    if pattern is None:
        return False, None
    assert pattern in ["megatron"], "Only megatron support gradient accumulation fusion currently"
    assert hasattr(b, "grad_added_to_main_grad"), "b.grad_added_to_main_grad must be set up before the backward pass."
    assert hasattr(b, "main_grad"), "b.main_grad must be set up before the backward pass."
    assert isinstance(b.main_grad, torch.Tensor) and b.main_grad.shape == b.shape, (
        "b.main_grad must be a tensor with the same shape as b"
    )
    b.grad_added_to_main_grad = True
    return True, b.main_grad


_dummy_wgrads: Dict[tuple, torch.Tensor] = {}


def _get_dummy_wgrad(shape, dtype: torch.dtype, zero: bool = False) -> torch.Tensor:
    """Cached placeholder gradient (contents never read) for weights whose real gradient
    went straight into ``main_grad``."""
    key = (tuple(shape), dtype)
    if key not in _dummy_wgrads:
        _dummy_wgrads[key] = torch.empty(shape, dtype=dtype, device="cuda", requires_grad=False)
    if zero:
        _dummy_wgrads[key].fill_(0)
    return _dummy_wgrads[key].detach()
