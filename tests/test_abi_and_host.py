"""CPU-side checks: the C-ABI library loads and exports every symbol the header declares,
argument validation works without a GPU, and the host layer mirrors the reference's
configs, op registration and fake (meta) kernels."""

import ctypes
import re
import subprocess
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "primus_turbo_amd.h"


def _declared():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"PT_API[^;(]*?\b(pt_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(native_lib):
    from primus_turbo import _native

    declared = _declared()
    assert len(declared) >= 13
    out = subprocess.run(["nm", "-D", "--defined-only", str(_native.LIB_PATH)], capture_output=True, text=True).stdout
    exported = set(re.findall(r" T (pt_[a-z0-9_]+)", out))
    assert set(declared) <= exported, sorted(set(declared) - exported)
    assert exported <= set(declared), f"exported but undeclared: {sorted(exported - set(declared))}"
    assert set(_native.exported_symbols()) == set(declared)
    for name in declared:
        assert isinstance(getattr(native_lib, name), ctypes._CFuncPtr)
    assert native_lib.pt_abi_version() >= 1


def test_header_compiles_as_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "primus_turbo_amd.h"\nint main(void){return PT_OK;}\n')
    r = subprocess.run(
        ["gcc", "-std=c99", "-Wall", "-Werror", "-I", str(HEADER.parent), "-c", str(src), "-o", str(tmp_path / "t.o")],
        capture_output=True,
        text=True,
    )
    assert r.returncode == 0, r.stderr


def test_argument_validation_without_gpu(native_lib):
    lib = native_lib
    # bad dtype codes / NULL pointers are rejected before anything is launched
    assert lib.pt_quantize_fp8_tensorwise(None, 9, 16, None, 3, None, None, None, 0, None) == -1
    assert b"bf16, fp16 or fp32" in lib.pt_last_error()
    assert lib.pt_quantize_fp8_tensorwise(None, 0, 16, None, 0, None, None, None, 0, None) == -1
    assert b"e4m3 or e5m2" in lib.pt_last_error()
    one = ctypes.c_float(0)
    assert lib.pt_quantize_fp8_tensorwise(1024, 0, 16, 2048, 3, None, ctypes.addressof(one), None, 0, None) == -3
    assert b"workspace" in lib.pt_last_error()
    assert lib.pt_quantize_fp8_tensorwise_static(None, 9, 16, None, 3, None, None, None, None) == -1
    assert lib.pt_quantize_fp8_tensorwise_static(1024, 0, 1 << 38, 2048, 3, None, ctypes.addressof(one), None, None) == -1
    assert b"MAX_NUMEL" in lib.pt_last_error()
    assert lib.pt_quantize_fp8_tensorwise_ex(1024, 0, 16, 2048, 3, None, ctypes.addressof(one), None, 0, None, 0, -1, None) == -1
    assert lib.pt_dequantize_fp8_tensorwise(None, 3, -1, None, None, 0, None) == -1
    assert lib.pt_quantize_fp8_rowwise(None, 0, 1, 1, 1, None, 7, None, None, None) == -1
    assert lib.pt_quantize_fp8_blockwise(None, 0, 8, 8, 3, None, None, None, None, None) == -1
    assert b"at least one" in lib.pt_last_error()
    assert lib.pt_quantize_fp8_blockwise_kmajor(1024, 0, 8, 8, 3, None, None, None, 0, None, None) == -1
    assert b"q_row" in lib.pt_last_error()
    # the gated grouped MX quantizer: act out of range, no row output, a Hadamard-transformed row direction
    assert lib.pt_glu_grouped_quantize_mx(1024, 0, 1024, None, 7, 8, 64, 3, 1024, None, 1024, 1, 1024, 1024, None, None, 0, 128, None) == -1
    assert b"act" in lib.pt_last_error()
    assert lib.pt_glu_grouped_quantize_mx(1024, 0, 1024, None, 0, 8, 64, 3, 1024, None, 1024, 1, None, None, 1024, 1024, 0, 128, None) == -1
    assert b"row direction" in lib.pt_last_error()
    assert lib.pt_glu_grouped_quantize_mx(1024, 0, 1024, None, 0, 8, 64, 3, 1024, None, 1024, 1, 1024, 1024, 1024, 1024, 4, 128, None) == -1
    assert lib.pt_dequantize_fp8_block(None, 3, 1, 8, 8, None, 0, 128, None, 0, None) == -1
    assert lib.pt_compute_group_offs(None, -1, 1, None, None, None) == -1
    assert lib.pt_quantize_fp8_tensorwise_workspace_bytes() >= 64


def test_ops_fail_loudly_on_cpu_tensors(native_lib):
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G

    x = torch.randn(8, 128).to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        turbo.ops.quantize_fp8(x, turbo.float8_e4m3, G.TENSORWISE)
    with pytest.raises(RuntimeError, match="no CPU path"):
        turbo.ops.quantize_fp8(x, turbo.float8_e4m3, G.ROWWISE, axis=-1)
    with pytest.raises(RuntimeError, match="no CPU path"):
        turbo.ops.quantize_fp8(x, turbo.float8_e4m3, G.BLOCKWISE, block_size=128, axis=1)
    with pytest.raises(AssertionError):
        turbo.ops.quantize_fp8(x, turbo.float8_e4m3, G.BLOCKWISE, axis=1)
    with pytest.raises(ValueError):
        turbo.ops.dequantize_fp8(x, torch.bfloat16, G.ROWWISE, scale_inv=x)


def test_missing_library_is_reported(monkeypatch, tmp_path):
    from primus_turbo import _native

    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(_native, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(RuntimeError, match="native library .* is missing"):
        _native.lib()


def test_configs_follow_the_reference_rules():
    from primus_turbo.pytorch.core.low_precision import (
        Float4QuantConfig,
        Float8QuantConfig,
        Format,
        ScaleDtype,
        ScalingGranularity,
        ScalingRecipe,
        ScalingStrategy,
    )

    c = Float8QuantConfig()
    assert (c.format, c.granularity, c.strategy, c.scale_dtype, c.block_size) == (
        Format.E4M3,
        ScalingGranularity.TENSORWISE,
        ScalingStrategy.DYNAMIC,
        ScaleDtype.FP32,
        None,
    )
    with pytest.raises(AssertionError, match="block_size must be set"):
        Float8QuantConfig(granularity=ScalingGranularity.BLOCKWISE)
    Float8QuantConfig(granularity=ScalingGranularity.BLOCKWISE, block_size=128)
    with pytest.raises(AssertionError):
        Float8QuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, block_size=128, scale_dtype=ScaleDtype.E8M0)
    with pytest.raises(AssertionError):
        Float8QuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, block_size=32)
    Float8QuantConfig(granularity=ScalingGranularity.MX_BLOCKWISE, block_size=32, scale_dtype=ScaleDtype.E8M0)
    f4 = Float4QuantConfig()
    assert f4.block_size == 32 and f4.scale_dtype == ScaleDtype.E8M0 and f4.format == Format.E2M1_X2
    with pytest.raises(AssertionError):
        Float4QuantConfig(block_size=16)
    with pytest.raises(AssertionError):
        Float4QuantConfig(granularity=ScalingGranularity.BLOCKWISE)
    assert ScalingRecipe() == (False, False, False, False, False)
    import primus_turbo.pytorch as turbo

    assert turbo.float8_e4m3 is torch.float8_e4m3fn and turbo.float8_e5m2 is torch.float8_e5m2


def test_fake_kernels_give_reference_shapes(native_lib):
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.core.low_precision import ScalingRecipe

    ext = torch.ops.primus_turbo_cpp_extension
    m = torch.empty(4, 300, 500, device="meta", dtype=torch.bfloat16)
    q, s = ext.quantize_fp8_tensorwise(m, torch.float8_e4m3fn, None)
    assert q.shape == m.shape and q.dtype == torch.float8_e4m3fn and s.shape == () and s.dtype == torch.float32
    for axis, want in ((0, (1, 300, 500)), (1, (4, 1, 500)), (-1, (4, 300, 1))):
        q, s = ext.quantize_fp8_rowwise(m, torch.float8_e5m2, axis, None)
        assert tuple(s.shape) == want
    assert ext.dequantize_fp8_tensorwise(q, s, torch.bfloat16).dtype == torch.bfloat16
    m2 = m[0]
    r = turbo.ops.quantize_fp8_with_trans(m2, torch.float8_e4m3fn, G.BLOCKWISE, block_size=128)
    assert [tuple(t.shape) for t in r] == [(300, 500), (300, 4), (300, 500), (3, 500)]
    q, s = turbo.ops.quantize_fp8(m, torch.float8_e4m3fn, G.BLOCKWISE, block_size=128, scaling_recipe=ScalingRecipe(True))
    assert tuple(s.shape) == (4, 3, 4)
    gl = torch.empty(6, device="meta", dtype=torch.int64)
    offs = ext.grouped_gemm_compute_offs(gl)
    assert tuple(offs.shape) == (7,)
    r = ext.quantize_fp8_blockwise_segment_m_row_col(m2, torch.float8_e4m3fn, 128, gl, offs)
    assert [tuple(t.shape) for t in r] == [(300, 500), (300 + 768, 500), (4, 300), (9, 500), (6,), (7,)]


def test_quantize_traces_under_torch_compile_on_meta():
    """The reference compiles quantize_fp8 with fullgraph=True; the op must be traceable."""
    import primus_turbo.pytorch as turbo  # noqa: F401
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode():
        x = torch.empty(64, 256, dtype=torch.bfloat16, device="cuda")
        q, s = torch.ops.primus_turbo_cpp_extension.quantize_fp8_tensorwise(x, torch.float8_e4m3fn, None)
        assert q.shape == (64, 256) and s.shape == ()
