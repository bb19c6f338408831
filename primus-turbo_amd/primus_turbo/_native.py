"""ctypes binding of libprimus_turbo_amd.so (the C-ABI library with the gfx950 kernels).

The library is the only compute backend: there is no CPU or eager fallback. If it
has not been built, every op raises ``RuntimeError`` naming the build command.
``import torch`` happens first so that the library binds to the HIP runtime that
PyTorch already loaded (one HIP runtime per process).
"""

from __future__ import annotations

import ctypes
import os
import threading
from pathlib import Path
from typing import Optional

import torch

_PKG_ROOT = Path(__file__).resolve().parent.parent  # .../primus-turbo_amd
LIB_PATH = Path(os.environ.get("PRIMUS_TURBO_AMD_LIB", _PKG_ROOT / "lib" / "libprimus_turbo_amd.so"))

# element type codes of include/primus_turbo_amd.h
DT_BF16, DT_F16, DT_F32, DT_E4M3, DT_E5M2, DT_E2M1X2, DT_E8M0 = range(7)

_DTYPE_CODE = {
    torch.bfloat16: DT_BF16,
    torch.float16: DT_F16,
    torch.float32: DT_F32,
    torch.float8_e4m3fn: DT_E4M3,
    torch.float8_e5m2: DT_E5M2,
}
if hasattr(torch, "float4_e2m1fn_x2"):
    _DTYPE_CODE[torch.float4_e2m1fn_x2] = DT_E2M1X2
if hasattr(torch, "float8_e8m0fnu"):
    _DTYPE_CODE[torch.float8_e8m0fnu] = DT_E8M0

_lib: Optional[ctypes.CDLL] = None
_lock = threading.Lock()

# status codes of include/primus_turbo_amd.h
PT_OK, PT_ERR_INVALID_ARGUMENT, PT_ERR_UNSUPPORTED, PT_ERR_WORKSPACE, PT_ERR_LAUNCH = 0, -1, -2, -3, -4

c_void_p, c_int, c_i64, c_size_t, c_float = (
    ctypes.c_void_p,
    ctypes.c_int,
    ctypes.c_int64,
    ctypes.c_size_t,
    ctypes.c_float,
)

# name -> (restype, argtypes); must match include/primus_turbo_amd.h
_SIGNATURES = {
    "pt_last_error": (ctypes.c_char_p, []),
    "pt_abi_version": (c_int, []),
    "pt_device_cu_count": (c_int, []),
    "pt_quantize_fp8_tensorwise_workspace_bytes": (c_size_t, []),
    "pt_quantize_fp8_tensorwise": (
        c_int,
        [c_void_p, c_int, c_i64, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "pt_quantize_fp8_tensorwise_ex": (
        c_int,
        [c_void_p, c_int, c_i64, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, ctypes.c_uint32,
         c_i64, c_void_p],
    ),
    "pt_quantize_fp8_tensorwise_static": (
        c_int,
        [c_void_p, c_int, c_i64, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "pt_tensorwise_static_release": (c_int, [c_void_p]),
    "pt_quantize_fp8_tensorwise_two_pass": (
        c_int,
        [c_void_p, c_int, c_i64, c_void_p, c_int, c_void_p, c_void_p, c_size_t, c_void_p],
    ),
    "pt_dequantize_fp8_tensorwise": (c_int, [c_void_p, c_int, c_i64, c_void_p, c_void_p, c_int, c_void_p]),
    "pt_quantize_fp8_rowwise": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_i64, c_void_p, c_int, c_void_p, c_void_p, c_void_p],
    ),
    "pt_dequantize_fp8_rowwise": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_i64, c_void_p, c_void_p, c_int, c_void_p],
    ),
    "pt_quantize_fp8_blockwise": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "pt_quantize_fp8_blockwise_t": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_void_p, c_void_p],
    ),
    "pt_quantize_fp8_blockwise_kmajor": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_int, c_void_p, c_void_p, c_void_p, c_i64, c_void_p, c_void_p],
    ),
    "pt_quantize_fp8_blockwise_weight": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_i64, c_void_p, c_int, c_void_p, c_void_p],
    ),
    "pt_quantize_fp8_blockwise_weight_dual": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_i64, c_void_p, c_void_p, c_i64, c_int, c_void_p, c_void_p],
    ),
    "pt_quantize_fp8_blockwise_segment_m_row_col_t": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_int, c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_void_p, c_void_p, c_i64,
         c_void_p, c_void_p],
    ),
    "pt_glu_quantize_fp8_blockwise_segment_m_row_col": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int, c_i64, c_i64, c_int, c_void_p, c_void_p, c_i64, c_void_p, c_void_p,
         c_void_p, c_void_p, c_i64, c_void_p, c_void_p],
    ),
    "pt_compute_group_offs": (c_int, [c_void_p, c_i64, c_i64, c_void_p, c_void_p, c_void_p]),
    "pt_quantize_fp8_blockwise_segment_m_row_col": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_int, c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p],
    ),
    "pt_gemm_fp8_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_int, c_int]),
    "pt_gemm_fp8": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_i64, c_i64, c_i64, c_int, c_int,
         c_int, c_i64, c_i64, c_i64, c_i64, c_int, c_int, c_int, c_void_p, c_size_t, c_int, c_void_p],
    ),
    "pt_glu_with_probs_fwd": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_int, c_void_p]),
    "pt_glu_with_probs_bwd": (
        c_int,
        [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_i64, c_i64, c_int, c_void_p],
    ),
    "pt_transpose_u8": (c_int, [c_void_p, c_void_p, c_i64, c_i64, c_i64, c_void_p]),
    "pt_transpose_2d": (c_int, [c_void_p, c_void_p, c_i64, c_i64, c_i64, c_int, c_void_p]),
    "pt_moe_permute_workspace_bytes": (c_size_t, [c_i64, c_i64]),
    "pt_moe_permute_preprocess": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_i64, c_i64, c_i64, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_size_t, c_void_p],
    ),
    "pt_moe_permute": (
        c_int,
        [c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_int, c_i64, c_void_p, c_i64, c_i64,
         c_i64, c_i64, c_void_p],
    ),
    "pt_moe_unpermute": (
        c_int,
        [c_void_p, c_void_p, c_int, c_i64, c_void_p, c_void_p, c_int, c_i64, c_void_p, c_i64, c_i64, c_i64, c_void_p],
    ),
    "pt_shuffle_mx_codes": (c_int, [c_void_p, c_void_p, c_i64, c_i64, c_int, c_void_p]),
    "pt_shuffle_e8m0_scale": (c_int, [c_void_p, c_void_p, c_i64, c_i64, c_i64, c_i64, c_i64, c_int, c_void_p]),
    "pt_gemm_mx_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_i64, c_i64, c_int]),
    "pt_gemm_mx": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_i64, c_i64, c_i64, c_i64, c_i64,
         c_i64, c_i64, c_int, c_void_p, c_size_t, c_int, c_void_p],
    ),
    "pt_quantize_mx": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_i64, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, ctypes.c_uint32,
         c_void_p],
    ),
    "pt_dequantize_mx": (c_int, [c_void_p, c_int, c_void_p, c_i64, c_i64, c_void_p, c_int, c_int, c_void_p]),
    "pt_grouped_gemm_fp8_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_i64, c_int]),
    "pt_grouped_gemm_fp8": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_i64, c_i64, c_i64, c_i64,
         c_i64, c_int, c_void_p, c_size_t, c_int, c_void_p],
    ),
    "pt_grouped_gemm_fp8_variable_k_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64]),
    "pt_grouped_gemm_fp8_variable_k": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_i64, c_i64, c_i64, c_i64,
         c_int, c_int, c_int, c_void_p, c_size_t, c_int, c_void_p],
    ),
    "pt_grouped_gemm_fp8_vec_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_i64, c_int]),
    "pt_grouped_gemm_fp8_vec": (
        c_int,
        [c_void_p, c_int, c_void_p, c_i64, c_void_p, c_int, c_void_p, c_i64, c_i64, c_void_p, c_int, c_void_p, c_i64, c_i64,
         c_i64, c_i64, c_i64, c_int, c_void_p, c_size_t, c_int, c_void_p],
    ),
    "pt_grouped_gemm_fp8_vec_variable_k_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_i64]),
    "pt_grouped_gemm_fp8_vec_variable_k": (
        c_int,
        [c_void_p, c_int, c_void_p, c_i64, c_void_p, c_int, c_void_p, c_i64, c_void_p, c_int, c_void_p, c_i64, c_i64, c_i64,
         c_i64, c_int, c_int, c_void_p, c_size_t, c_int, c_void_p],
    ),
    "pt_grouped_quantize_mx": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_int, c_void_p, c_void_p, c_void_p, c_i64, c_void_p, c_void_p, c_int, c_void_p,
         c_void_p, c_int, c_i64, ctypes.c_uint32, c_void_p],
    ),
    "pt_glu_grouped_quantize_mx": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int, c_i64, c_i64, c_int, c_void_p, c_void_p, c_void_p, c_i64, c_void_p,
         c_void_p, c_void_p, c_void_p, c_int, c_i64, c_void_p],
    ),
    "pt_grouped_gemm_mx": (
        c_int,
        [c_void_p, c_int, c_void_p, c_i64, c_i64, c_void_p, c_int, c_void_p, c_i64, c_i64, c_void_p, c_int, c_void_p,
         c_void_p, c_i64, c_i64, c_i64, c_i64, c_i64, c_void_p, c_size_t, c_int, c_void_p],
    ),
    "pt_grouped_gemm_mx_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64, c_i64]),
    "pt_grouped_gemm_mx_variable_k_workspace_bytes": (c_size_t, [c_i64, c_i64, c_i64]),
    "pt_grouped_gemm_mx_variable_k": (
        c_int,
        [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_i64, c_i64, c_i64, c_i64, c_int,
         c_void_p, c_size_t, c_int, c_void_p],
    ),
    "pt_dequantize_fp8_block": (
        c_int,
        [c_void_p, c_int, c_i64, c_i64, c_i64, c_void_p, c_i64, c_i64, c_void_p, c_int, c_void_p],
    ),
}


def exported_symbols():
    """Names every build of the library must export (used by the load test)."""
    return sorted(_SIGNATURES)


def lib() -> ctypes.CDLL:
    """Load (once) and return the native library; raise loudly if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"primus_turbo: native library {LIB_PATH} is missing. Build it with "
                f"`python {_PKG_ROOT / 'build_native.py'}` (hipcc, --offload-arch=gfx950). "
                "There is no CPU fallback."
            )
        handle = ctypes.CDLL(str(LIB_PATH))
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the build is stale
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError(f"primus_turbo: dtype {dtype} is not supported by the gfx950 kernels") from None


def check(status: int) -> None:
    if status != 0:
        msg = lib().pt_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"primus_turbo native error {status}: {msg}")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def stream_of(t: torch.Tensor) -> int:
    """Raw hipStream_t of torch's current stream on ``t``'s device. Kernels are launched on the
    current device, so that has to be the tensor's."""
    if t.device.index != torch.cuda.current_device():
        raise RuntimeError(
            f"primus_turbo: tensor on {t.device} but the current device is cuda:{torch.cuda.current_device()}; "
            "wrap the call in torch.cuda.device(tensor.device)"
        )
    return torch.cuda.current_stream(t.device).cuda_stream


def require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "primus_turbo: tensors must live on a ROCm GPU (the kernels are gfx950 HIP; there is no CPU path)"
            )


# ---------------------------------------------------------------------------
# Zero-filled device workspace for one launch. Not kept between calls: a buffer that outlives the
# call would have to live outside the private memory pool of whatever graph capture, or warm-up
# run for one, happens to be active -- torch.compile's CUDA-graph trees insist that nothing
# allocated there stays alive -- and an op cannot tell. Only the fallback of the tensorwise
# quantizer uses it (its normal path keeps the exchange words in the library's static scratch).
# ---------------------------------------------------------------------------
def zeroed_workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    return torch.zeros(max(nbytes, 256), dtype=torch.uint8, device=device)
