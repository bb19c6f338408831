"""``primus_turbo.pytorch``: the low-precision op surface on gfx950 HIP kernels."""

import torch  # noqa: F401  (loads the HIP runtime the native library binds to)

import primus_turbo.pytorch.ops  # noqa: F401
import primus_turbo.pytorch.kernels.quantization.mx_dispatcher_ops  # noqa: F401  (registers the reference's MX op names)
from primus_turbo.pytorch.core import low_precision

float8_e4m3 = low_precision.float8_e4m3
float8_e5m2 = low_precision.float8_e5m2
float4_e2m1fn_x2 = low_precision.float4_e2m1fn_x2
