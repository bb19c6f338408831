"""Committed golden vectors: replayed by the oracle on the CPU and by the HIP kernels on the GPU."""

import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import formats as F

GOLD = Path(__file__).parent / "golden" / "quant_golden.npz"


@pytest.fixture(scope="module")
def gold():
    return dict(np.load(GOLD, allow_pickle=False))


def test_oracle_reproduces_golden(gold):
    sys.path.insert(0, str(GOLD.parent))
    import make_golden

    fresh = make_golden.build()
    assert sorted(fresh) == sorted(gold)
    for k, v in fresh.items():
        assert v.dtype == gold[k].dtype and v.shape == gold[k].shape, k
        assert np.ascontiguousarray(v).tobytes() == np.ascontiguousarray(gold[k]).tobytes(), k


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int32).numpy().view(np.uint32)


def _codes(t):
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


@pytest.mark.gpu
def test_hip_reproduces_golden_fp8(gold, native_lib):
    import primus_turbo.pytorch as turbo
    from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G
    from primus_turbo.pytorch.core.low_precision import ScalingRecipe
    from primus_turbo.pytorch.kernels.quantization.quantization_impl import (
        quant_fp8_blockwise_segment_m_row_col_impl as seg,
    )

    x = torch.from_numpy(F.bf16_bits_to_f32(gold["x_bf16_bits"])).to(torch.bfloat16).cuda()
    for fmt, dt in (("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)):
        q, s = turbo.ops.quantize_fp8(x, dt, G.TENSORWISE)
        assert np.array_equal(_codes(q), gold[f"tensorwise_{fmt}_q"])
        assert _bits(s) == gold[f"tensorwise_{fmt}_sinv"].view(np.uint32)
        for axis in (0, 1):
            q, s = turbo.ops.quantize_fp8(x, dt, G.ROWWISE, axis=axis)
            assert np.array_equal(_codes(q), gold[f"rowwise{axis}_{fmt}_q"])
            assert np.array_equal(_bits(s), gold[f"rowwise{axis}_{fmt}_sinv"].view(np.uint32))
        qr, sr, qc, sc = turbo.ops.quantize_fp8_with_trans(x, dt, G.BLOCKWISE, block_size=128)
        assert np.array_equal(_codes(qr), gold[f"block_row_{fmt}_q"])
        assert np.array_equal(_codes(qc), gold[f"block_col_{fmt}_q"])
        assert np.array_equal(_bits(sr), gold[f"block_row_{fmt}_sinv"].view(np.uint32))
        assert np.array_equal(_bits(sc), gold[f"block_col_{fmt}_sinv"].view(np.uint32))
        q, s = turbo.ops.quantize_fp8(x, dt, G.BLOCKWISE, block_size=128, scaling_recipe=ScalingRecipe(True))
        assert np.array_equal(_codes(q), gold[f"block_weight_{fmt}_q"])
        assert np.array_equal(_bits(s), gold[f"block_weight_{fmt}_sinv"].view(np.uint32))
    gl = torch.from_numpy(gold["group_lens"]).cuda()
    offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(gl)
    qr, qc, sr, sc, _, poffs = seg(x, torch.float8_e4m3fn, 128, gl, offs, None)
    w = int(gold["segment_padded_offs"][-1])
    assert np.array_equal(poffs.cpu().numpy(), gold["segment_padded_offs"])
    assert np.array_equal(_codes(qr), gold["segment_row_q"])
    assert np.array_equal(_bits(sr), gold["segment_row_sinv"].view(np.uint32))
    assert np.array_equal(_codes(qc)[:w], gold["segment_col_q"])
    assert np.array_equal(_bits(sc)[: w // 128], gold["segment_col_sinv"].view(np.uint32))


@pytest.mark.gpu
def test_hip_reproduces_golden_mx(gold, native_lib):
    from primus_turbo.pytorch.core.low_precision import ScalingRecipe
    from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

    x = torch.from_numpy(F.bf16_bits_to_f32(gold["x_bf16_bits"])).to(torch.bfloat16).cuda()
    fmts = [("e4m3", torch.float8_e4m3fn, qi.quantize_mxfp8_impl), ("e5m2", torch.float8_e5m2, qi.quantize_mxfp8_impl)]
    if hasattr(torch, "float4_e2m1fn_x2"):
        fmts.append(("e2m1", torch.float4_e2m1fn_x2, qi.quantize_mxfp4_impl))
    for fmt, dt, fn in fmts:
        for two_d in (False, True):
            tag = f"mx_{fmt}_{'2d' if two_d else '1d'}"
            rec = ScalingRecipe(use_2d_block=two_d)
            rq, rs, cq, cs = fn(x, dt, None, 32, with_trans=True, scaling_recipe=rec, scaling_recipe_for_trans=rec)
            assert np.array_equal(_codes(rq), gold[f"{tag}_row_q"]), tag
            assert np.array_equal(_codes(rs), gold[f"{tag}_row_scale"]), tag
            assert np.array_equal(_codes(cq), gold[f"{tag}_col_q"]), tag
            assert np.array_equal(_codes(cs), gold[f"{tag}_col_scale"]), tag
