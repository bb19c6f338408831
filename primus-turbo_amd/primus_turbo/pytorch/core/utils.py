"""Device queries used by the low-precision ops."""

from __future__ import annotations

import functools
from typing import Tuple

import torch


@functools.lru_cache(maxsize=None)
def _capability(index: int) -> Tuple[int, int]:
    p = torch.cuda.get_device_properties(index)
    return (p.major, p.minor)


def get_device_compute_capability() -> Tuple[int, int]:
    """(major, minor) of the current GPU; (9, 5) is gfx950."""
    return _capability(torch.cuda.current_device())


def is_gfx950() -> bool:
    return torch.cuda.is_available() and get_device_compute_capability() == (9, 5)


def is_gfx942() -> bool:
    return torch.cuda.is_available() and get_device_compute_capability() == (9, 4)


def is_gfx1250() -> bool:
    return torch.cuda.is_available() and get_device_compute_capability() == (12, 5)


@functools.lru_cache(maxsize=None)
def _num_cus(index: int) -> int:
    return torch.cuda.get_device_properties(index).multi_processor_count


def get_num_cus() -> int:
    return _num_cus(torch.cuda.current_device())
