"""CPU restatement of the pre-shuffled MX operand layouts (TEST INFRASTRUCTURE ONLY; only tests
may import it).

The index maps are those of /root/reference/csrc/include/primus_turbo/device/shuffle.cuh:39-48
(scales) and :62-80 (codes); shapes, padding (rows to 256, columns to 8, pad byte 0) and the
in-range checks follow /root/reference/csrc/pytorch/shuffle/shuffle.cpp:31-44 and
/root/reference/csrc/kernels/shuffle/shuffle.cu:32-78. Bytes only: parity is bit-exact.
Pinned in tests/test_oracle_shuffle.py against the reshape / axis-permutation statement of the
same layouts (the form in which AITER publishes them: ``shuffle_weight`` with layout (16, 16) and
``e8m0_shuffle``), against hand-computed offsets and as bijections."""

from __future__ import annotations

import numpy as np


def shuffled_code_offsets(rows: int, row_bytes: int) -> np.ndarray:
    """``[rows, row_bytes]`` -> offset of every byte in the shuffled tensor (shuffle.cuh:62-80)."""
    assert rows % 16 == 0 and row_bytes % 32 == 0
    r, c = np.indices((rows, row_bytes), dtype=np.int64)
    in_blk = c & 31
    return (r >> 4) * (row_bytes << 4) + (c >> 5) * 512 + (in_blk >> 4) * 256 + (r & 15) * 16 + (in_blk & 15)


def shuffle_codes(codes: np.ndarray) -> np.ndarray:
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.size, dtype=np.uint8)
    out[shuffled_code_offsets(*codes.shape).ravel()] = codes.ravel()
    return out.reshape(codes.shape)


def unshuffle_codes(shuffled: np.ndarray) -> np.ndarray:
    shuffled = np.ascontiguousarray(shuffled, dtype=np.uint8)
    return shuffled.ravel()[shuffled_code_offsets(*shuffled.shape)]


def scale_pad_shape(M: int, N: int):
    """shuffle.cpp:31-34: rows padded to 256, columns to 8."""
    return -(-M // 256) * 256, -(-N // 8) * 8


def shuffled_scale_offsets(M: int, N: int, N_pad: int) -> np.ndarray:
    """``[M, N]`` -> offset of every scale byte in the shuffled ``[M_pad, N_pad]`` tensor
    (shuffle.cuh:39-48)."""
    row, col = np.indices((M, N), dtype=np.int64)
    i0, i1, i2 = row >> 5, (row >> 4) & 1, row & 15
    i3, i4, i5 = col >> 3, (col >> 2) & 1, col & 3
    return i0 * (N_pad >> 3) * 256 + i3 * 256 + i5 * 64 + i2 * 4 + i4 * 2 + i1


def shuffle_scale(scale: np.ndarray) -> np.ndarray:
    """``[M, N]`` E8M0 bytes -> shuffled ``[M_pad, N_pad]``, zero where there is no scale."""
    scale = np.ascontiguousarray(scale, dtype=np.uint8)
    M, N = scale.shape
    Mp, Np = scale_pad_shape(M, N)
    out = np.zeros(Mp * Np, dtype=np.uint8)
    out[shuffled_scale_offsets(M, N, Np).ravel()] = scale.ravel()
    return out.reshape(Mp, Np)


def unshuffle_scale(shuffled: np.ndarray, M: int, N: int) -> np.ndarray:
    shuffled = np.ascontiguousarray(shuffled, dtype=np.uint8)
    return shuffled.ravel()[shuffled_scale_offsets(M, N, shuffled.shape[1])]
