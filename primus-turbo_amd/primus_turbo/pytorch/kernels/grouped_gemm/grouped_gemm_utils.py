"""Group offset helper (reference: primus_turbo/pytorch/kernels/grouped_gemm/grouped_gemm_utils.py:28-34)."""

from __future__ import annotations

import torch


def group_offs_from_lens(group_lens: torch.Tensor) -> torch.Tensor:
    """``[G]`` int64 group lengths -> ``[G + 1]`` int64 exclusive prefix sums, on the device,
    without a host synchronisation."""
    return torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(group_lens)
