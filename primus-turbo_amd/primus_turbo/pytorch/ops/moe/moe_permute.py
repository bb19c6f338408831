"""``moe_permute`` / ``moe_unpermute``: token rows into expert-major order for the grouped GEMMs of an
MoE expert bank and back, with autograd (interface of the reference's
primus_turbo/pytorch/ops/moe/moe_permute.py:16-456: same arguments, outputs and error behaviour).

``moe_permute`` returns ``(permuted_tokens, row_id_map, tokens_per_expert, overflow_flag,
num_dispatched_tokens, permuted_scaling_factor, permuted_probs)``; its backward is the unpermute
(sum over a token's experts) and ``moe_unpermute``'s backward is the permute. With
``num_permuted_tokens <= 0`` the size of the permuted tensor is read back from the device
(``tokens_per_expert.sum()``), as in the reference; a positive value keeps the op free of host
synchronisation."""

from __future__ import annotations

from typing import Optional, Tuple

import torch

import primus_turbo.pytorch.kernels.moe.moe_permute_impl  # noqa: F401  (registers the dispatcher ops)

__all__ = ["moe_permute", "moe_unpermute"]

_ops = torch.ops.primus_turbo_cpp_extension


class _MoEPermute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, tokens, expert_map, num_local_experts, num_topk, pad_multiple=0, num_permuted_tokens=-1,
                scaling_factor=None, probs=None, scales_per_token=0, use_fp8=False, probs_topk_stride=0):
        dev = tokens.device
        T, hidden = int(tokens.shape[0]), int(tokens.shape[-1])
        stride = int(probs_topk_stride) if probs is not None else 0
        ctx.meta = (T, hidden, num_local_experts, use_fp8, probs is not None,
                    probs.dtype if probs is not None else None, stride, stride if stride > 0 else num_local_experts)
        if use_fp8 and scaling_factor is not None:
            assert scales_per_token > 0, "scales_per_token must be > 0 when use_fp8=True"
        assert not (use_fp8 and probs is not None and tokens.requires_grad), (
            "moe_permute: FP8 + probs backward is unsupported"
        )
        with_sf = use_fp8 and scaling_factor is not None
        if T == 0:  # nothing dispatched to this rank
            row_id_map = torch.zeros((pad_multiple, 2 * num_local_experts + 1), dtype=torch.int32, device=dev)
            tokens_per_expert = torch.zeros((num_local_experts,), dtype=torch.int64, device=dev)
            overflow_flag = torch.zeros((1,), dtype=torch.int32, device=dev)
            num_dispatched = torch.zeros((1,), dtype=torch.int32, device=dev)
            out = tokens.new_empty((0, hidden))
            out_sf = scaling_factor.new_empty((0, scales_per_token)) if with_sf else None
            out_probs = probs.new_zeros((0,)) if probs is not None else None
        else:
            row_id_map, tokens_per_expert, overflow_flag, num_dispatched = _ops.permute_preprocessing(
                expert_map, num_local_experts, num_topk, pad_multiple, num_permuted_tokens, stride)
            rows = int(num_permuted_tokens) if num_permuted_tokens > 0 else int(tokens_per_expert.sum().item())
            out = torch.empty((rows, hidden), dtype=tokens.dtype, device=dev)
            out_sf = torch.empty((rows, scales_per_token), dtype=scaling_factor.dtype, device=dev) if with_sf else None
            out_probs = torch.empty((rows,), dtype=probs.dtype, device=dev) if probs is not None else None
            _ops.permute(tokens.contiguous(), out, scaling_factor, out_sf, None if probs is None else probs.contiguous(),
                         out_probs, row_id_map, num_dispatched, pad_multiple, num_local_experts, hidden,
                         scales_per_token, use_fp8, probs is not None, rows, stride)
        ctx.save_for_backward(row_id_map, num_dispatched)
        ctx.mark_non_differentiable(row_id_map, tokens_per_expert, overflow_flag, num_dispatched)
        if out_sf is not None:
            ctx.mark_non_differentiable(out_sf)
        return out, row_id_map, tokens_per_expert, overflow_flag, num_dispatched, out_sf, out_probs

    @staticmethod
    def backward(ctx, grad_permuted, _map, _tpe, _flag, _nd, _sf, grad_permuted_probs):
        T, hidden, E, use_fp8, with_probs, probs_dtype, stride, row_width = ctx.meta
        assert not use_fp8, "_MoEPermute.backward: FP8 backward not supported"
        row_id_map, num_dispatched = ctx.saved_tensors
        grad_permuted = grad_permuted.contiguous()
        grad_tokens = torch.empty((T, hidden), dtype=grad_permuted.dtype, device=grad_permuted.device)
        grad_probs = None
        if with_probs and grad_permuted_probs is not None:
            grad_permuted_probs = grad_permuted_probs.contiguous()
            grad_probs = torch.empty((T, row_width), dtype=probs_dtype, device=grad_permuted.device)
        else:
            grad_permuted_probs = None
        if T > 0:
            _ops.unpermute(grad_permuted, grad_tokens, grad_permuted_probs, grad_probs, row_id_map, num_dispatched, E,
                           hidden, grad_probs is not None, stride)
        return grad_tokens, None, None, None, None, None, None, grad_probs, None, None, None


class _MoEUnpermute(torch.autograd.Function):
    @staticmethod
    def forward(ctx, permuted_tokens, row_id_map, num_dispatched_tokens_tensor, restore_shape, num_local_experts,
                permuted_probs, probs_topk_stride, pad_multiple):
        dev = permuted_tokens.device
        rows = int(permuted_tokens.shape[0])
        T, hidden = int(restore_shape[0]), int(restore_shape[1])
        row_width = probs_topk_stride if probs_topk_stride > 0 else num_local_experts
        ctx.meta = (rows, hidden, num_local_experts, permuted_probs is not None,
                    permuted_probs.dtype if permuted_probs is not None else None, probs_topk_stride, pad_multiple)
        # the kernel writes every row (zeros for a token routed nowhere); without it the result is zero
        alloc = torch.empty if (rows > 0 and T > 0) else torch.zeros
        tokens = alloc((T, hidden), dtype=permuted_tokens.dtype, device=dev)
        probs = alloc((T, row_width), dtype=permuted_probs.dtype, device=dev) if permuted_probs is not None else None
        if rows > 0 and T > 0:
            _ops.unpermute(permuted_tokens.contiguous(), tokens,
                           None if permuted_probs is None else permuted_probs.contiguous(), probs, row_id_map,
                           num_dispatched_tokens_tensor, num_local_experts, hidden, permuted_probs is not None,
                           probs_topk_stride)
        ctx.save_for_backward(row_id_map, num_dispatched_tokens_tensor)
        return tokens, probs

    @staticmethod
    def backward(ctx, grad_tokens, grad_probs):
        rows, hidden, E, with_probs, probs_dtype, stride, pad_multiple = ctx.meta
        row_id_map, num_dispatched = ctx.saved_tensors
        grad_tokens = grad_tokens.contiguous()
        dev = grad_tokens.device
        # rows that no map entry names (beyond the experts' padded ranges) carry no gradient
        grad_permuted = torch.zeros((rows, hidden), dtype=grad_tokens.dtype, device=dev)
        grad_permuted_probs = None
        if with_probs and grad_probs is not None:
            grad_probs = grad_probs.contiguous()
            grad_permuted_probs = torch.zeros((rows,), dtype=probs_dtype, device=dev)
        else:
            grad_probs = None
        if rows > 0 and grad_tokens.shape[0] > 0:
            _ops.permute(grad_tokens, grad_permuted, None, None, grad_probs, grad_permuted_probs, row_id_map,
                         num_dispatched, pad_multiple, E, hidden, 0, False, grad_permuted_probs is not None, rows,
                         stride)
        return grad_permuted, None, None, None, None, grad_permuted_probs, None, None


def moe_permute(
    tokens: torch.Tensor,
    expert_map: torch.Tensor,
    *,
    num_local_experts: int,
    num_topk: int = 0,
    pad_multiple: int = 0,
    num_permuted_tokens: int = -1,
    scaling_factor: Optional[torch.Tensor] = None,
    probs: Optional[torch.Tensor] = None,
    probs_layout: str = "topk",
    scales_per_token: int = 0,
    use_fp8: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, Optional[torch.Tensor],
           Optional[torch.Tensor]]:
    """Permute ``tokens [T, hidden]`` into expert-major order.

    ``expert_map``: bool routing map ``[T, num_local_experts]`` or ``topk_idx [T, num_topk]``
    (int32 / int64, entries outside the local experts ignored). Every expert's rows are padded with
    zero rows to a multiple of ``pad_multiple``. ``probs`` is ``[T, num_local_experts]``
    (``probs_layout="routing_map"``) or ``[T, num_topk]`` aligned with ``topk_idx`` (``"topk"``);
    ``scaling_factor [T, scales_per_token]`` rides along with FP8 tokens (``use_fp8``)."""
    if probs_layout not in ("routing_map", "topk"):
        raise ValueError(f"moe_permute: probs_layout must be 'routing_map' or 'topk', got {probs_layout!r}")
    if probs_layout == "topk" and num_topk <= 0:
        raise ValueError("moe_permute: probs_layout='topk' requires num_topk > 0")
    stride = num_topk if probs_layout == "topk" else 0
    return _MoEPermute.apply(tokens, expert_map, num_local_experts, num_topk, pad_multiple, num_permuted_tokens,
                             scaling_factor, probs, scales_per_token, use_fp8, stride)


def moe_unpermute(
    permuted_tokens: torch.Tensor,
    row_id_map: torch.Tensor,
    num_dispatched_tokens_tensor: torch.Tensor,
    *,
    restore_shape: torch.Size,
    num_local_experts: int,
    permuted_probs: Optional[torch.Tensor] = None,
    probs_topk_stride: int = 0,
    pad_multiple: int = 0,
) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Inverse of :func:`moe_permute`: ``tokens[t]`` = sum of the token's rows in ``permuted_tokens``,
    shape ``restore_shape``; ``permuted_probs`` come back as ``[T, num_local_experts]``
    (``probs_topk_stride=0``) or ``[T, probs_topk_stride]``. ``pad_multiple`` must be the one the map
    was made with (backward writes the zero rows through it)."""
    return _MoEUnpermute.apply(permuted_tokens, row_id_map, num_dispatched_tokens_tensor, restore_shape,
                               num_local_experts, permuted_probs, probs_topk_stride, pad_multiple)
