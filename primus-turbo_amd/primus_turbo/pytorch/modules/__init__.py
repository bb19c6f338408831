"""Modules on top of the low-precision ops (the callers of the hot path that the reference ships
in ``primus_turbo/pytorch/modules``; only the FP8 linear layer belongs to this build)."""

from .linear_fp8 import Float8Linear

__all__ = ["Float8Linear"]
