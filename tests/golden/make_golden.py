"""Writes tests/golden/quant_golden.npz: one seeded 64 x 256 bf16 tile (with outliers, an
all-zero block and a tiny-magnitude block) and the bytes / scales every quantizer of the
path must produce for it.

The reference holds no golden vectors for these ops and cannot be run in this build, so
the expected outputs come from the CPU oracle (oracle/quantize.py), which is pinned on its
own by tests/test_oracle_*.py. The fixture freezes those answers: the oracle test replays
them on the CPU and the GPU tests compare the HIP kernels with the same bytes.

    python tests/golden/make_golden.py
"""

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import formats as F  # noqa: E402
from oracle import quantize as Q  # noqa: E402

GROUP_LENS = np.array([40, 0, 24], dtype=np.int64)


def make_input() -> np.ndarray:
    rng = np.random.default_rng(20251125)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    idx = rng.choice(x.size, 16, replace=False)
    x.reshape(-1)[idx] *= 100.0
    x[5, 32:64] = 0.0  # an all-zero 32-block
    x[9, 128:256] = 3e-6 * rng.standard_normal(128)  # below the blockwise eps
    return F.f32_to_bf16_bits(x)


def build() -> dict:
    xb = make_input()
    x = F.bf16_bits_to_f32(xb)
    out = {"x_bf16_bits": xb, "group_lens": GROUP_LENS}
    for fmt in ("e4m3", "e5m2"):
        q, s = Q.fp8_tensorwise(x, fmt)
        out[f"tensorwise_{fmt}_q"], out[f"tensorwise_{fmt}_sinv"] = q, s
        for axis in (0, 1):
            q, s = Q.fp8_rowwise(x, axis, fmt)
            out[f"rowwise{axis}_{fmt}_q"], out[f"rowwise{axis}_{fmt}_sinv"] = q, s
        qr, sr, qc, sc = Q.fp8_blockwise_dual(x, fmt)
        out[f"block_row_{fmt}_q"], out[f"block_row_{fmt}_sinv"] = qr, sr
        out[f"block_col_{fmt}_q"], out[f"block_col_{fmt}_sinv"] = qc, sc
        q, s = Q.fp8_blockwise_weight(x, fmt)
        out[f"block_weight_{fmt}_q"], out[f"block_weight_{fmt}_sinv"] = q, s
    seg = Q.fp8_blockwise_segment_m_row_col(x, GROUP_LENS, "e4m3")
    w = seg["written_rows"]
    out["segment_row_q"], out["segment_row_sinv"] = seg["row"], seg["row_scale"]
    out["segment_col_q"], out["segment_col_sinv"] = seg["col"][:w], seg["col_scale"][: w // 128]
    out["segment_padded_offs"] = seg["padded_offs"]
    for fmt in ("e4m3", "e5m2", "e2m1"):
        for two_d in (False, True):
            tag = f"mx_{fmt}_{'2d' if two_d else '1d'}"
            q, s = Q.mx_quant_rowwise(x, fmt, two_d)
            out[f"{tag}_row_q"], out[f"{tag}_row_scale"] = q, s
            q, s = Q.mx_quant_colwise(x, fmt, two_d)
            out[f"{tag}_col_q"], out[f"{tag}_col_scale"] = q, s
    return out


if __name__ == "__main__":
    data = build()
    path = Path(__file__).with_name("quant_golden.npz")
    np.savez_compressed(path, **data)
    print(f"wrote {path} ({path.stat().st_size} bytes, {len(data)} arrays)")
