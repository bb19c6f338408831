"""MoE permute impl layer: the reference's dispatcher ops ``permute_preprocessing`` / ``permute`` /
``unpermute`` (schemas csrc/pytorch/bindings_pytorch.cpp:100-112, bodies
csrc/pytorch/moe_permute/moe_permute.cpp:42-282) registered from Python on the gfx950 kernels behind
``pt_moe_permute_preprocess`` / ``pt_moe_permute`` / ``pt_moe_unpermute``. The output arguments of
``permute`` / ``unpermute`` are declared as mutated so that ``torch.compile`` keeps the calls."""

from __future__ import annotations

from typing import Optional

import torch

from primus_turbo import _native as N

_lib = torch.library.Library("primus_turbo_cpp_extension", "FRAGMENT")

_MAP_KIND = {torch.bool: 0, torch.int32: 1, torch.int64: 2}


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


_lib.define(
    "permute_preprocessing(Tensor expert_map, int num_local_experts, int num_topk, int pad_multiple, "
    "int num_permuted_tokens, int probs_topk_stride=0) -> (Tensor, Tensor, Tensor, Tensor)"
)


def _preprocessing_outputs(expert_map, num_local_experts, pad_multiple):
    dev, T = expert_map.device, expert_map.shape[0]
    # entries that no token uses stay zero (the reference leaves them uninitialised)
    row_id_map = torch.zeros((T + pad_multiple, 2 * num_local_experts + 1), dtype=torch.int32, device=dev)
    tokens_per_expert = torch.empty((num_local_experts,), dtype=torch.int64, device=dev)
    overflow_flag = torch.empty((1,), dtype=torch.int32, device=dev)
    num_dispatched = torch.zeros((1,), dtype=torch.int32, device=dev)
    return row_id_map, tokens_per_expert, overflow_flag, num_dispatched


def _permute_preprocessing(expert_map: torch.Tensor, num_local_experts: int, num_topk: int, pad_multiple: int,
                           num_permuted_tokens: int, probs_topk_stride: int = 0):
    N.require_cuda(expert_map)
    _check(expert_map.dtype in _MAP_KIND, "expert_map must be bool or int or int64")
    _check(expert_map.dim() == 2, "expert_map must be 2D")
    _check(expert_map.is_contiguous(), "expert_map must be contiguous")
    if expert_map.dtype == torch.bool:
        _check(expert_map.shape[1] == num_local_experts, "bool expert_map second dimension must equal num_local_experts")
        _check(probs_topk_stride == 0,
               "probs_topk_stride > 0 (topk-aligned probs) requires the topk_idx expert_map code path; "
               "routing_map mode only supports multihot probs")
    else:
        _check(expert_map.shape[1] == num_topk, "index expert_map second dimension must equal num_topk")
        _check(probs_topk_stride in (0, num_topk),
               "probs_topk_stride must be 0 (multihot probs) or equal to num_topk (topk-aligned probs)")
    _check(expert_map.shape[0] > 0, "permute_preprocessing needs at least one token")
    outs = _preprocessing_outputs(expert_map, num_local_experts, pad_multiple)
    row_id_map, tokens_per_expert, overflow_flag, num_dispatched = outs
    lib = N.lib()
    ws_bytes = lib.pt_moe_permute_workspace_bytes(expert_map.shape[0], num_local_experts)
    ws = torch.empty(max(ws_bytes, 4), dtype=torch.uint8, device=expert_map.device)
    N.check(lib.pt_moe_permute_preprocess(
        N.ptr(expert_map), _MAP_KIND[expert_map.dtype], expert_map.shape[0], num_local_experts, num_topk, pad_multiple,
        num_permuted_tokens, int(probs_topk_stride > 0), N.ptr(row_id_map), N.ptr(tokens_per_expert),
        N.ptr(overflow_flag), N.ptr(num_dispatched), N.ptr(ws), ws.numel(), N.stream_of(expert_map)))
    return outs


def _permute_preprocessing_meta(expert_map, num_local_experts, num_topk, pad_multiple, num_permuted_tokens,
                                probs_topk_stride=0):
    return _preprocessing_outputs(expert_map, num_local_experts, pad_multiple)


_lib.impl("permute_preprocessing", _permute_preprocessing, "CUDA")
_lib.impl("permute_preprocessing", _permute_preprocessing, "CPU")  # raises: no CPU path
_lib.impl("permute_preprocessing", _permute_preprocessing_meta, "Meta")

_lib.define(
    "permute(Tensor tokens, Tensor(a!) output_tokens, Tensor? scaling_factor, Tensor(b!)? output_scaling_factor, "
    "Tensor? probs, Tensor(c!)? output_probs, Tensor row_id_map, Tensor num_dispatched_token_tensor, "
    "int pad_multiple, int num_local_experts, int hidden_size, int scales_per_token, bool use_fp8, bool with_probs, "
    "int num_permuted_token, int probs_stride=0) -> ()"
)


def _check_map(row_id_map, num_dispatched, num_local_experts, what):
    _check(row_id_map.is_cuda and row_id_map.dtype == torch.int32 and row_id_map.is_contiguous(),
           f"{what}: row_id_map must be contiguous int32 CUDA tensor")
    _check(row_id_map.dim() == 2 and row_id_map.shape[1] == 2 * num_local_experts + 1,
           f"{what}: row_id_map must be [rows, 2 * num_local_experts + 1]")
    _check(num_dispatched.is_cuda and num_dispatched.dtype == torch.int32 and num_dispatched.numel() == 1,
           f"{what}: num_dispatched_token_tensor must be contiguous int32 CUDA tensor with exactly one element")


def _probs_args(probs, out_probs, probs_stride, num_local_experts, what):
    if probs is None:
        return None, None, 0, 0
    _check(out_probs is not None, f"{what}: with_probs=true but probs / output_probs not provided")
    _check(probs.dtype == out_probs.dtype and probs.element_size() in (2, 4), f"{what}: probs must be 2- or 4-byte floats")
    _check(probs.is_contiguous() and out_probs.is_contiguous(), f"{what}: probs must be contiguous")
    return probs, out_probs, probs.element_size(), probs_stride if probs_stride > 0 else num_local_experts


def _permute(tokens, output_tokens, scaling_factor, output_scaling_factor, probs, output_probs, row_id_map,
             num_dispatched_token_tensor, pad_multiple: int, num_local_experts: int, hidden_size: int,
             scales_per_token: int, use_fp8: bool, with_probs: bool, num_permuted_token: int, probs_stride: int = 0) -> None:
    _check(num_permuted_token >= 0, "num_permuted_token must be >= 0")
    if num_permuted_token == 0:
        return
    _check(probs_stride >= 0, "probs_stride must be >= 0")
    N.require_cuda(tokens, output_tokens)
    _check(tokens.is_contiguous() and output_tokens.is_contiguous(), "permute: tokens / output_tokens must be contiguous")
    _check(tokens.dim() == 2 and output_tokens.dim() == 2, "permute: tokens / output_tokens must be 2D")
    _check(tokens.shape[1] == hidden_size, "permute: tokens.shape[1] must equal hidden_size")
    _check(tuple(output_tokens.shape) == (num_permuted_token, hidden_size) and output_tokens.dtype == tokens.dtype,
           "permute: output_tokens shape must be [num_permuted_token, hidden_size]")
    _check_map(row_id_map, num_dispatched_token_tensor, num_local_experts, "permute")
    _check(row_id_map.shape[0] == tokens.shape[0] + pad_multiple, "permute: row_id_map must hold one row per token plus "
           "pad_multiple padding rows")
    sf = out_sf = None
    sf_bytes = 0
    if use_fp8 and scaling_factor is not None:
        _check(output_scaling_factor is not None, "permute: use_fp8 needs output_scaling_factor")
        _check(scales_per_token > 0 and tuple(scaling_factor.shape) == (tokens.shape[0], scales_per_token),
               "permute: scaling_factor must be [num_tokens, scales_per_token]")
        _check(tuple(output_scaling_factor.shape) == (num_permuted_token, scales_per_token)
               and output_scaling_factor.dtype == scaling_factor.dtype, "permute: output_scaling_factor shape mismatch")
        sf, out_sf = scaling_factor.contiguous(), output_scaling_factor
        sf_bytes = scales_per_token * scaling_factor.element_size()
    p, out_p, p_bytes, p_stride = _probs_args(probs if with_probs else None, output_probs, probs_stride,
                                              num_local_experts, "permute")
    if p is not None:
        _check(p.numel() == tokens.shape[0] * p_stride, "permute: probs must hold probs_stride values per token")
        _check(out_p.numel() == num_permuted_token, "permute: output_probs must be [num_permuted_token]")
    N.check(N.lib().pt_moe_permute(
        N.ptr(tokens), N.ptr(output_tokens), hidden_size * tokens.element_size(), N.ptr(sf), N.ptr(out_sf), sf_bytes,
        N.ptr(p), N.ptr(out_p), p_bytes, p_stride, N.ptr(row_id_map), tokens.shape[0], pad_multiple, num_local_experts,
        num_permuted_token, N.stream_of(tokens)))


_lib.impl("permute", _permute, "CUDA")
_lib.impl("permute", _permute, "CPU")
_lib.impl("permute", lambda *a, **k: None, "Meta")

_lib.define(
    "unpermute(Tensor permuted_tokens, Tensor(a!) output_tokens, Tensor? permuted_probs, Tensor(b!)? output_probs, "
    "Tensor row_id_map, Tensor num_dispatched_tokens_tensor, int num_local_experts, int hidden_size, bool with_probs, "
    "int probs_stride=0) -> ()"
)


def _unpermute(permuted_tokens, output_tokens, permuted_probs, output_probs, row_id_map, num_dispatched_tokens_tensor,
               num_local_experts: int, hidden_size: int, with_probs: bool, probs_stride: int = 0) -> None:
    N.require_cuda(permuted_tokens, output_tokens)
    _check(permuted_tokens.dtype in (torch.bfloat16, torch.float16) and output_tokens.dtype == permuted_tokens.dtype,
           "unpermute: tokens must be bfloat16 or float16")
    _check(permuted_tokens.is_contiguous() and output_tokens.is_contiguous(), "unpermute: tokens must be contiguous")
    _check(permuted_tokens.dim() == 2 and output_tokens.dim() == 2 and permuted_tokens.shape[1] == hidden_size
           and output_tokens.shape[1] == hidden_size, "unpermute: tokens must be [rows, hidden_size]")
    _check_map(row_id_map, num_dispatched_tokens_tensor, num_local_experts, "unpermute")
    _check(row_id_map.shape[0] >= output_tokens.shape[0], "unpermute: row_id_map has fewer rows than output_tokens")
    p, out_p, p_bytes, p_stride = _probs_args(permuted_probs if with_probs else None, output_probs, probs_stride,
                                              num_local_experts, "unpermute")
    if p is not None:
        _check(p.numel() == permuted_tokens.shape[0], "unpermute: permuted_probs must hold one value per permuted row")
        _check(out_p.numel() == output_tokens.shape[0] * p_stride, "unpermute: output_probs must hold probs_stride values per token")
    N.check(N.lib().pt_moe_unpermute(
        N.ptr(permuted_tokens), N.ptr(output_tokens), N.dtype_code(permuted_tokens.dtype), hidden_size, N.ptr(p),
        N.ptr(out_p), p_bytes, p_stride, N.ptr(row_id_map), output_tokens.shape[0], num_local_experts,
        permuted_tokens.shape[0], N.stream_of(permuted_tokens)))


_lib.impl("unpermute", _unpermute, "CUDA")
_lib.impl("unpermute", _unpermute, "CPU")
_lib.impl("unpermute", lambda *a, **k: None, "Meta")
