"""Bit-level number formats of the low-precision path (TEST INFRASTRUCTURE ONLY).

This package is the checker for the HIP kernels: only ``tests/``,
``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline leg may import it.
Nothing under ``primus-turbo_amd/`` imports it and it is never a fallback.

Formats restated here (OCP encodings, which is what gfx950 uses —
/root/reference/primus_turbo/pytorch/core/low_precision.py:77-83,
/root/reference/csrc/include/primus_turbo/float8.h:35-45):

* E4M3 (``float8_e4m3fn``): bias 7, 3 mantissa bits, max finite 448 (0x7E),
  no infinities, 0x7F/0xFF = NaN.
* E5M2 (``float8_e5m2``): bias 15, 2 mantissa bits, max finite 57344 (0x7B).
* E2M1: bias 1, 1 mantissa bit, values +-{0, .5, 1, 1.5, 2, 3, 4, 6}.
* E8M0: one biased exponent byte, value 2^(b-127).

The encoders round to nearest, ties to even, and expect inputs already clamped
to the finite range (the reference clamps before every cast:
/root/reference/csrc/include/primus_turbo/device/quant_utils.cuh:33-40).

How these are pinned (see tests/test_oracle_formats.py): the FP8 encoders and
decoders are compared exhaustively against torch's CPU casts
(``Tensor.to(torch.float8_e4m3fn)`` / ``float8_e5m2``) over every bf16 bit
pattern and dense fp32 grids with exact ties; E2M1 against the 16-entry value
table and every midpoint; E8M0 against ``torch.float8_e8m0fnu``.
"""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np


@dataclass(frozen=True)
class MiniFloat:
    name: str
    exp_bits: int
    man_bits: int
    bias: int
    max_finite: float

    @property
    def min_normal_exp(self) -> int:
        return 1 - self.bias


E4M3 = MiniFloat("e4m3", 4, 3, 7, 448.0)
E5M2 = MiniFloat("e5m2", 5, 2, 15, 57344.0)
E2M1 = MiniFloat("e2m1", 2, 1, 1, 6.0)


def encode_rne(x: np.ndarray, fmt: MiniFloat) -> np.ndarray:
    """Round finite values (|x| <= fmt.max_finite) to the nearest code, ties to even.

    ``x`` may be float32 or float64; the arithmetic below is exact in either
    (only power-of-two scalings and ``rint`` of values below 2^5).
    Returns uint8 codes with the sign in the top bit of the format's width.
    """
    x = np.asarray(x)
    if x.dtype not in (np.float32, np.float64):
        x = x.astype(np.float32)
    a = np.abs(x).astype(np.float64)
    if np.any(~np.isfinite(a)) or np.any(a > fmt.max_finite):
        raise ValueError("encode_rne expects values clamped to the finite range")
    sign = np.signbit(x).astype(np.uint8) << (fmt.exp_bits + fmt.man_bits)

    m, e = np.frexp(a)  # a = m * 2^e, m in [0.5, 1)
    unb = e - 1  # floor(log2 a) for a > 0
    normal = (a > 0) & (unb >= fmt.min_normal_exp)
    steps = 1 << fmt.man_bits

    # normal numbers: significand m*2 in [1, 2) -> n = rint(m * 2 * steps) in [steps, 2*steps]
    n_norm = np.rint(m * (2 * steps)).astype(np.int64)
    carry = n_norm == 2 * steps
    n_norm = np.where(carry, steps, n_norm)
    exp_field = (unb + fmt.bias + carry.astype(np.int64)).astype(np.int64)
    code_norm = (exp_field << fmt.man_bits) | (n_norm - steps)

    # subnormals: quantum 2^(min_normal_exp - man_bits); a result of `steps` is the
    # smallest normal and its code is exactly that integer
    quantum = 2.0 ** (fmt.min_normal_exp - fmt.man_bits)
    code_sub = np.rint(a / quantum).astype(np.int64)

    code = np.where(normal, code_norm, code_sub).astype(np.uint8)
    return (code | sign).astype(np.uint8)


def decode_table(fmt: MiniFloat) -> np.ndarray:
    """float32 value of every code (index = code). NaN/Inf codes follow OCP."""
    width = 1 + fmt.exp_bits + fmt.man_bits
    out = np.zeros(1 << width, dtype=np.float32)
    for code in range(1 << width):
        s = -1.0 if (code >> (width - 1)) & 1 else 1.0
        ef = (code >> fmt.man_bits) & ((1 << fmt.exp_bits) - 1)
        mf = code & ((1 << fmt.man_bits) - 1)
        if ef == 0:
            v = mf * 2.0 ** (fmt.min_normal_exp - fmt.man_bits)
        else:
            v = (1.0 + mf / (1 << fmt.man_bits)) * 2.0 ** (ef - fmt.bias)
        if fmt is E4M3 and ef == 15 and mf == 7:
            v = float("nan")
        if fmt is E5M2 and ef == 31:
            v = float("inf") if mf == 0 else float("nan")
        out[code] = s * v
    return out


_TABLES: dict[str, np.ndarray] = {}


def decode(codes: np.ndarray, fmt: MiniFloat) -> np.ndarray:
    if fmt.name not in _TABLES:
        _TABLES[fmt.name] = decode_table(fmt)
    return _TABLES[fmt.name][np.asarray(codes, dtype=np.uint8)]


# ---------------------------------------------------------------------------
# E8M0 shared exponents
# ---------------------------------------------------------------------------
# (val_to_add, target_max_pow2) per element format
# /root/reference/primus_turbo/flydsl/quantization/mxfp8_quant_flydsl.py:44-66 (E4M3: 1<<19, 135-127=8;
# E5M2: 1<<20, 142-127=15), /root/reference/primus_turbo/flydsl/quantization/mxfp4_quant_kernel.py:78-89
# (E2M1: 1<<21, 2).
E8M0_RULE = {"e4m3": (1 << 19, 8), "e5m2": (1 << 20, 15), "e2m1": (1 << 21, 2)}


def e8m0_exponent(amax: np.ndarray, fmt: MiniFloat) -> np.ndarray:
    """Unbiased shared exponent e (int32, in [-127, 128]) for a block whose abs-max is ``amax``.

    e = clamp((((bits(amax) + val_to_add) >> 23) & 0x1FF) - 127 - target_pow2, -127, 128),
    all in 32-bit integers. The E8M0 byte is e + 127.
    """
    add, tgt = E8M0_RULE[fmt.name]
    bits = np.asarray(amax, dtype=np.float32).view(np.uint32).astype(np.int64)
    ext = ((bits + add) >> 23) & 0x1FF
    e = ext - 127 - tgt
    return np.clip(e, -127, 128).astype(np.int32)


def e8m0_to_f32(byte: np.ndarray) -> np.ndarray:
    """Scale value used by the de-quantizers: the byte placed in the fp32 exponent field
    (/root/reference/csrc/include/primus_turbo/device/utils.cuh:124-126). Byte 0 gives 0.0
    and byte 255 gives +inf, unlike the arithmetic value 2^(b-127)."""
    return (np.asarray(byte, dtype=np.uint8).astype(np.uint32) << 23).view(np.float32)


# ---------------------------------------------------------------------------
# bf16 helpers (numpy has no bf16)
# ---------------------------------------------------------------------------
def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16 bit patterns (NaN stays NaN)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    r = np.where(nan, (u >> 16) | 0x40, r)
    return r.astype(np.uint16)
