"""Backend names of the reference API, kept so that callers which pin or query a backend
keep working. This build has exactly one backend per op (the gfx950 HIP kernels), so the
selection machinery of the reference (primus_turbo/pytorch/core/backend.py:86-624: user
choice > env > auto-tune > default > first capable) collapses to "the native kernel";
choices are recorded and otherwise ignored."""

from __future__ import annotations

import os
from dataclasses import dataclass
from enum import Enum, auto
from typing import Dict, Optional

ENV_GEMM_BACKEND = "PRIMUS_TURBO_GEMM_BACKEND"
ENV_GROUPED_GEMM_BACKEND = "PRIMUS_TURBO_GROUPED_GEMM_BACKEND"
ENV_AUTO_TUNE = "PRIMUS_TURBO_AUTO_TUNE"


class PrecisionType(Enum):
    FP4 = auto()
    FP8 = auto()
    BF16_FP16_FP32 = auto()


class BackendType(Enum):
    CK = auto()
    HIPBLASLT = auto()
    AITER = auto()
    TRITON = auto()
    DEEP_EP = auto()
    TURBO = auto()
    FLYDSL = auto()
    HIPKITTENS = auto()


@dataclass
class BackendChoice:
    backend: Optional[BackendType] = None
    auto_tune: bool = False


class GlobalBackendManager:
    """Records backend requests; every request resolves to the native gfx950 kernels."""

    _gemm: Dict[PrecisionType, BackendChoice] = {}
    _grouped_gemm: Dict[PrecisionType, BackendChoice] = {}

    @classmethod
    def set_gemm_backend(cls, backend: Optional[BackendType] = None, precision: PrecisionType = PrecisionType.FP8,
                         auto_tune: bool = False) -> None:
        cls._gemm[precision] = BackendChoice(backend, auto_tune)

    @classmethod
    def set_grouped_gemm_backend(cls, backend: Optional[BackendType] = None,
                                 precision: PrecisionType = PrecisionType.FP8, auto_tune: bool = False) -> None:
        cls._grouped_gemm[precision] = BackendChoice(backend, auto_tune)

    @classmethod
    def get_gemm_backend(cls, precision: PrecisionType) -> BackendChoice:
        return cls._gemm.get(precision, BackendChoice())

    @classmethod
    def get_grouped_gemm_backend(cls, precision: PrecisionType) -> BackendChoice:
        return cls._grouped_gemm.get(precision, BackendChoice())

    @classmethod
    def auto_tune_enabled(cls) -> bool:
        return os.environ.get(ENV_AUTO_TUNE, "0") == "1"

    @classmethod
    def reset(cls) -> None:
        cls._gemm.clear()
        cls._grouped_gemm.clear()
