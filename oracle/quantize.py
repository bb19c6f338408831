"""CPU restatement of the reference quantizers (TEST INFRASTRUCTURE ONLY).

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s CPU-baseline leg
may import this module; the product never routes through it.

Inputs are numpy float32 arrays holding the exact values of the bf16/fp16/fp32
source (widening is exact). All scale arithmetic is IEEE fp32 like the device
kernels (reference build flags carry no fast-math: /root/reference/setup.py:297-326).
Outputs are uint8 code arrays and float32 / uint8 scale arrays.

What each function follows, and what pins it (tests/test_oracle_*.py):

* ``fp8_tensorwise`` / ``fp8_rowwise`` — device semantics of
  /root/reference/csrc/pytorch/quantization/quantization.cpp:44-208 with
  /root/reference/csrc/include/primus_turbo/device/quant_utils.cuh:33-74
  (fp32 multiply; eps 1e-12). Pinned by closed forms (all-zero tensor, single
  spike, power-of-two amax), by the pure-PyTorch formula of
  /root/reference/tests/pytorch/ref/quantization_ref.py:31-58 on fp32 input (where
  that formula and the device semantics coincide bit for bit), and by torch's own
  CPU fp8 cast for the rounding.
* ``fp8_blockwise`` / ``fp8_blockwise_dual`` / ``fp8_blockwise_weight`` /
  ``fp8_blockwise_segment_m_row_col`` — /root/reference/primus_turbo/triton/quantization/quant_blockwise.py:11-327
  and /root/reference/csrc/kernels/quantization/quantization_blockwise.cu:18-346
  (eps 1e-4, stores 1/scale). Pinned by invariants: every block holds a code of
  magnitude qmax, dual == two single-axis calls, grouped row scales == plain 1x128
  scales transposed, padded rows are zero bytes, brute-force per-block python loop.
* ``mxfp8`` / ``mxfp4`` — integer E8M0 rule and exact power-of-two scaling of
  /root/reference/primus_turbo/flydsl/quantization/mxfp8_quant_flydsl.py:44-66,337-525 and
  /root/reference/primus_turbo/flydsl/quantization/mxfp4_quant_kernel.py:78-89,121-149;
  shapes and padding of /root/reference/csrc/pytorch/quantization/quantization.cpp:511-969.
  The HIP sources of the reference MX quantizers are absent from the snapshot, so
  bit-identity with them is PARITY UNPINNED; what is pinned is the published rule:
  brute force over every bf16 amax, the saturation invariant, 2-D blocks constant
  over 32x32 tiles, round trips through the de-quantizer. ``hadamard16`` restates the
  recipe's fixed 16-point Hadamard transform (``use_rht``; pinned against scipy's
  Sylvester matrix and by its involution, rounding order PARITY UNPINNED as above).
  Stochastic rounding is not restated (random by design: the tests check its properties).
* ``mx_grouped_quant`` — per-group composition of the two above in the padded layouts of
  /root/reference/csrc/pytorch/quantization/quantization.cpp:971-1100 (rows of a group padded
  to 32 / 128 with zero data); pinned by the group-by-group round trip against the dense
  quantizer and by the zero-pad invariants (same PARITY UNPINNED remark for bit-identity
  with the reference's own kernels). Its 2-D blocks are counted from each group's first row,
  pad rows carrying their block's exponent: the reference's grouped kernels are absent, so
  this placement is PARITY UNPINNED; pinned is that each group's slice equals the dense 2-D
  quantizer of that group's rows.
"""

from __future__ import annotations

import numpy as np

from .formats import E2M1, E4M3, E5M2, MiniFloat, decode, e8m0_exponent, e8m0_to_f32, encode_rne

F32 = np.float32


def _fmt(name_or_fmt) -> MiniFloat:
    if isinstance(name_or_fmt, MiniFloat):
        return name_or_fmt
    return {"e4m3": E4M3, "e5m2": E5M2, "e2m1": E2M1}[name_or_fmt]


def _cdiv(a: int, b: int) -> int:
    return (a + b - 1) // b


def _scale_from_amax(amax: np.ndarray, qmax: float, eps: float):
    """scale = qmax / max(amax, eps); scale_inv = 1.0f / scale — fp32, IEEE division."""
    with np.errstate(divide="ignore", over="ignore"):
        amax = np.maximum(np.asarray(amax, dtype=F32), F32(eps))
        scale = (F32(qmax) / amax).astype(F32)
        scale_inv = (F32(1.0) / scale).astype(F32)
    return scale, scale_inv


def _abs_max(x: np.ndarray, axis=None, keepdims=False) -> np.ndarray:
    """abs-max that ignores NaN like fmaxf does; empty reductions give 0."""
    a = np.abs(x)
    a = np.where(np.isnan(a), F32(0), a)
    if a.size == 0:
        shape = list(a.shape)
        if axis is None:
            return F32(0)
        shape[axis] = 1
        out = np.zeros(shape, dtype=F32)
        return out if keepdims else np.squeeze(out, axis=axis)
    return np.max(a, axis=axis, keepdims=keepdims).astype(F32)


def _cast_fp8(x: np.ndarray, scale: np.ndarray, fmt: MiniFloat) -> np.ndarray:
    """fp8_rne(fmax(fmin(x*scale, qmax), -qmax)); NaN -> +qmax as fminf drops the NaN."""
    qmax = F32(fmt.max_finite)
    with np.errstate(over="ignore", invalid="ignore"):
        v = (x.astype(F32) * scale).astype(F32)
    v = np.where(np.isnan(v), qmax, v)
    v = np.clip(v, -qmax, qmax)
    return encode_rne(v, fmt)


# ---------------------------------------------------------------------------
# tensorwise / rowwise
# ---------------------------------------------------------------------------
def fp8_tensorwise(x: np.ndarray, fmt="e4m3", scale: np.ndarray | None = None):
    """-> (codes uint8 like x, scale_inv float32 0-dim)."""
    fmt = _fmt(fmt)
    x = np.asarray(x, dtype=F32)
    if scale is None:
        scale_v, scale_inv = _scale_from_amax(_abs_max(x), fmt.max_finite, 1e-12)
    else:
        scale_v = np.asarray(scale, dtype=F32).reshape(())
        with np.errstate(divide="ignore"):
            scale_inv = (F32(1.0) / scale_v).astype(F32)
    return _cast_fp8(x, scale_v, fmt), np.asarray(scale_inv, dtype=F32).reshape(())


def fp8_rowwise(x: np.ndarray, axis: int, fmt="e4m3"):
    """One scale per slice along ``axis`` -> (codes, scale_inv with that axis kept as 1)."""
    fmt = _fmt(fmt)
    x = np.asarray(x, dtype=F32)
    axis = axis if axis >= 0 else x.ndim + axis
    amax = _abs_max(x, axis=axis, keepdims=True)
    scale, scale_inv = _scale_from_amax(amax, fmt.max_finite, 1e-12)
    return _cast_fp8(x, scale, fmt), scale_inv


def fp8_dequant(codes: np.ndarray, scale_inv: np.ndarray, fmt="e4m3") -> np.ndarray:
    """float(q) * scale_inv in fp32 (broadcast); the caller rounds to the output dtype."""
    with np.errstate(over="ignore", invalid="ignore"):
        return (decode(codes, _fmt(fmt)) * np.asarray(scale_inv, dtype=F32)).astype(F32)


# ---------------------------------------------------------------------------
# 128-blockwise (fp32 scales, eps 1e-4)
# ---------------------------------------------------------------------------
def _pad2d(x: np.ndarray, bm: int, bn: int) -> np.ndarray:
    M, N = x.shape
    out = np.zeros((_cdiv(M, bm) * bm, _cdiv(N, bn) * bn), dtype=F32)
    out[:M, :N] = x
    return out


def fp8_blockwise(x: np.ndarray, axis: int, fmt="e4m3", block: int = 128):
    """1-D blocks along ``axis`` of a 2-D tensor.

    axis 1: scale_inv [M, cdiv(N, block)]; axis 0: scale_inv [cdiv(M, block), N].
    Partial edge blocks see zeros for the missing elements.
    """
    fmt = _fmt(fmt)
    x = np.asarray(x, dtype=F32)
    M, N = x.shape
    axis = axis % 2
    if axis == 1:
        xp = _pad2d(x, 1, block).reshape(M, -1, block)
        amax = _abs_max(xp, axis=2, keepdims=True)
        scale, scale_inv = _scale_from_amax(amax, fmt.max_finite, 1e-4)
        codes = _cast_fp8(xp, scale, fmt).reshape(M, -1)[:, :N]
        return codes, scale_inv.reshape(M, -1)
    xp = _pad2d(x, block, 1).reshape(-1, block, N)
    amax = _abs_max(xp, axis=1, keepdims=True)
    scale, scale_inv = _scale_from_amax(amax, fmt.max_finite, 1e-4)
    codes = _cast_fp8(xp, scale, fmt).reshape(-1, N)[:M, :]
    return codes, scale_inv.reshape(-1, N)


def fp8_blockwise_dual(x: np.ndarray, fmt="e4m3", block: int = 128):
    """-> (row codes, row scale_inv [M, N/b], col codes, col scale_inv [M/b, N])."""
    r, rs = fp8_blockwise(x, 1, fmt, block)
    c, cs = fp8_blockwise(x, 0, fmt, block)
    return r, rs, c, cs


def fp8_blockwise_weight(w: np.ndarray, fmt="e4m3", block: int = 128):
    """One scale per block x block tile of a 2-D or 3-D weight.

    -> (codes like w, scale_inv [..., cdiv(M, block), cdiv(N, block)]).
    """
    fmt = _fmt(fmt)
    w = np.asarray(w, dtype=F32)
    squeeze = w.ndim == 2
    if squeeze:
        w = w[None]
    B, M, N = w.shape
    mb, nb = _cdiv(M, block), _cdiv(N, block)
    wp = np.zeros((B, mb * block, nb * block), dtype=F32)
    wp[:, :M, :N] = w
    t = wp.reshape(B, mb, block, nb, block)
    amax = _abs_max(_abs_max(t, axis=4, keepdims=True), axis=2, keepdims=True)
    scale, scale_inv = _scale_from_amax(amax, fmt.max_finite, 1e-4)
    codes = _cast_fp8(t, scale, fmt).reshape(B, mb * block, nb * block)[:, :M, :N]
    scale_inv = scale_inv.reshape(B, mb, nb)
    if squeeze:
        return codes[0], scale_inv[0]
    return codes, scale_inv


def fp8_blockwise_dequant(codes, scale_inv, axis: int, fmt="e4m3", block: int = 128):
    codes = np.asarray(codes)
    M, N = codes.shape
    s = np.asarray(scale_inv, dtype=F32)
    if axis % 2 == 1:
        full = np.repeat(s, block, axis=1)[:, :N]
    else:
        full = np.repeat(s, block, axis=0)[:M, :]
    return (decode(codes, _fmt(fmt)) * full).astype(F32)


def fp8_blockwise_weight_dequant(codes, scale_inv, fmt="e4m3", block: int = 128):
    codes = np.asarray(codes)
    s = np.asarray(scale_inv, dtype=F32)
    M, N = codes.shape[-2:]
    full = np.repeat(np.repeat(s, block, axis=-2), block, axis=-1)[..., :M, :N]
    return (decode(codes, _fmt(fmt)) * full).astype(F32)


def padded_group_offs(group_lens: np.ndarray, block: int = 128):
    """Each group length rounded up to ``block`` -> (padded_lens [G], padded_offs [G+1]) int64."""
    gl = np.asarray(group_lens, dtype=np.int64)
    pl = ((gl + block - 1) // block) * block
    po = np.zeros(len(gl) + 1, dtype=np.int64)
    po[1:] = np.cumsum(pl)
    return pl, po


def group_offs(group_lens: np.ndarray) -> np.ndarray:
    gl = np.asarray(group_lens, dtype=np.int64)
    o = np.zeros(len(gl) + 1, dtype=np.int64)
    o[1:] = np.cumsum(gl)
    return o


def fp8_blockwise_segment_m_row_col(x: np.ndarray, group_lens: np.ndarray, fmt="e4m3", block: int = 128):
    """Fused grouped quantizer of a packed-M activation ``x [M, N]``.

    Returns a dict with
      row        uint8 [M, N]            1 x block row quant of every input row
      row_scale  f32   [cdiv(N,b), M]    its 1/scale, stored transposed
      col        uint8 [M + G*b, N]      block x 1 column quant of the segment-padded
                                         tensor (each group starts on a multiple of b,
                                         pad rows are zero data -> code 0)
      col_scale  f32   [(M+G*b)/b, N]
      padded_lens int64 [G], padded_offs int64 [G+1]
      written_rows  number of leading rows of ``col`` / row-blocks of ``col_scale`` the
                    kernel defines (= padded_offs[-1]); the rest is unspecified memory.
    """
    fmt = _fmt(fmt)
    x = np.asarray(x, dtype=F32)
    M, N = x.shape
    gl = np.asarray(group_lens, dtype=np.int64)
    G = len(gl)
    offs = group_offs(gl)
    pl, po = padded_group_offs(gl, block)
    row, rs = fp8_blockwise(x, 1, fmt, block)
    Mp_max = M + G * block
    col = np.zeros((Mp_max, N), dtype=np.uint8)
    col_scale = np.zeros((_cdiv(Mp_max, block), N), dtype=F32)
    for g in range(G):
        n = int(gl[g])
        if n == 0:
            continue
        seg = np.zeros((int(pl[g]), N), dtype=F32)
        seg[:n] = x[offs[g] : offs[g] + n]
        c, cs = fp8_blockwise(seg, 0, fmt, block)
        col[po[g] : po[g + 1]] = c
        col_scale[po[g] // block : po[g + 1] // block] = cs
    return dict(
        row=row,
        row_scale=np.ascontiguousarray(rs.T),
        col=col,
        col_scale=col_scale,
        padded_lens=pl,
        padded_offs=po,
        written_rows=int(po[-1]),
    )


# ---------------------------------------------------------------------------
# MX (E8M0 shared exponent per 32 elements)
# ---------------------------------------------------------------------------
def _mx_scale_and_cast(blocks: np.ndarray, amax: np.ndarray, fmt: MiniFloat):
    """blocks [..., 32] float32, amax broadcastable -> (codes uint8, e8m0 byte uint8)."""
    e = e8m0_exponent(amax, fmt)
    byte = (e + 127).astype(np.uint8)
    # x * 2^-e is exact except for results below the fp32 normal range, which round to a
    # zero code in every target format; float64 keeps the product exact here.
    y = blocks.astype(np.float64) * np.exp2(-e.astype(np.float64))
    qmax = fmt.max_finite
    y = np.where(np.isnan(y), qmax, y)
    y = np.clip(y, -qmax, qmax)
    return encode_rne(y, fmt), byte


def _pack_fp4(codes: np.ndarray) -> np.ndarray:
    """Pairs along the last axis: element 2p -> low nibble, 2p+1 -> high nibble of byte p
    (/root/reference/csrc/kernels/quantization/dequantization_mxfp4.cu:110-113)."""
    lo = codes[..., 0::2].astype(np.uint8)
    hi = codes[..., 1::2].astype(np.uint8)
    return (lo | (hi << 4)).astype(np.uint8)


def unpack_fp4(packed: np.ndarray) -> np.ndarray:
    p = np.asarray(packed, dtype=np.uint8)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 2,), dtype=np.uint8)
    out[..., 0::2] = p & 0xF
    out[..., 1::2] = p >> 4
    return out


def hadamard16(v: np.ndarray) -> np.ndarray:
    """The fixed 16-point Hadamard transform of the MXFP4 recipe along the last axis (length a
    multiple of 16, transformed in groups of 16), in fp32 with the operation order of
    /root/reference/primus_turbo/flydsl/quantization/mxfp4_quant_kernel.py:92-118: an H4 butterfly
    inside each run of four elements, an H4 butterfly across the four runs, times 0.25 -- i.e.
    (H4 (x) H4) / 4, the orthonormal Sylvester matrix of order 16. There are no random signs:
    the transform is its own inverse and cancels between two operands that both carry it.
    Pinned against scipy's Sylvester matrix on inputs where fp32 is exact, by the involution, and
    bit for bit against a one-operation-at-a-time evaluation of the FlyDSL text on data whose
    rounding depends on the order (tests/test_oracle_gemm.py). Bit-identity of the rounding order
    with the reference's HIP kernel is PARITY UNPINNED (its source is absent); the FlyDSL text
    states that the two agree."""
    v = np.asarray(v, dtype=F32)
    g = v.reshape(v.shape[:-1] + (v.shape[-1] // 16, 4, 4))  # [.., group, block, local]

    def h4(v0, v1, v2, v3):
        a0, a1, a2, a3 = (v0 + v1).astype(F32), (v0 - v1).astype(F32), (v2 + v3).astype(F32), (v2 - v3).astype(F32)
        return (a0 + a2).astype(F32), (a1 + a3).astype(F32), (a0 - a2).astype(F32), (a1 - a3).astype(F32)

    with np.errstate(over="ignore", invalid="ignore"):
        o = np.stack(h4(g[..., 0], g[..., 1], g[..., 2], g[..., 3]), axis=-1)       # within each block
        r = np.stack(h4(o[..., 0, :], o[..., 1, :], o[..., 2, :], o[..., 3, :]), axis=-2)  # across the blocks
        r = (r * F32(0.25)).astype(F32)
    return r.reshape(v.shape)


def mx_quant_rowwise(x: np.ndarray, fmt, use_2d_block: bool = False, pad: int = 128, use_rht: bool = False):
    """MX quantization along the last axis of a 2-D ``x [M, K]``.

    -> (codes [M, K_pad] (FP4: packed [M, K_pad/2]), e8m0 bytes [M, K_pad/32]) with
    K_pad = K rounded up to ``pad``; the K padding is zero data (scale byte 0 for a
    fully padded block). With ``use_2d_block`` one exponent is shared by each 32x32
    tile (rows beyond M count as zeros) and replicated into the scale slot of each of
    its rows. ``use_rht`` (MXFP4 recipe): every 16 consecutive elements (of the zero-padded
    row) go through ``hadamard16`` first; abs-max, scale and codes are those of the
    transformed values (mxfp4_quant_kernel.py:176-199).
    """
    fmt = _fmt(fmt)
    x = np.asarray(x, dtype=F32)
    M, K = x.shape
    Kp = _cdiv(K, pad) * pad
    xp = np.zeros((M, Kp), dtype=F32)
    xp[:, :K] = x
    if use_rht:
        assert not use_2d_block, "the recipe never combines 2-D blocks with the Hadamard transform"
        xp = hadamard16(xp)
    blk = xp.reshape(M, Kp // 32, 32)
    if use_2d_block:
        Mp = _cdiv(M, 32) * 32
        a = np.zeros((Mp, Kp // 32), dtype=F32)
        a[:M] = _abs_max(blk, axis=2)
        a = _abs_max(a.reshape(Mp // 32, 32, Kp // 32), axis=1, keepdims=True)
        amax = np.broadcast_to(a, (Mp // 32, 32, Kp // 32)).reshape(Mp, Kp // 32)[:M, :, None]
    else:
        amax = _abs_max(blk, axis=2, keepdims=True)
    codes, byte = _mx_scale_and_cast(blk, amax, fmt)
    codes = codes.reshape(M, Kp)
    if fmt is E2M1:
        codes = _pack_fp4(codes)
    return codes, byte.reshape(M, Kp // 32)


def mx_quant_colwise(x: np.ndarray, fmt, use_2d_block: bool = False, pad: int = 128, use_rht: bool = False):
    """MX quantization along axis 0 of ``x [M, K]``, emitted transposed:
    codes [K, M_pad] (FP4 packed [K, M_pad/2]) and bytes [K, M_pad/32]."""
    x = np.asarray(x, dtype=F32)
    return mx_quant_rowwise(np.ascontiguousarray(x.T), fmt, use_2d_block, pad, use_rht)


def mx_grouped_quant(x: np.ndarray, group_lens: np.ndarray, fmt, row_align: int = 32, col_align: int = 128,
                     row_rht: bool = False, col_rht: bool = False, row_2d: bool = False, col_2d: bool = False):
    """Grouped MX quantizer of a packed-M activation ``x [M, N]`` (layout rules of
    /root/reference/csrc/pytorch/quantization/quantization.cpp:971-1100 and
    /root/reference/primus_turbo/pytorch/kernels/quantization/quantization_impl.py:572-700:
    every group is virtually zero-padded along M, to ``row_align`` rows for the row direction
    and to ``col_align`` rows for the column direction; per-block numerics are those of the
    dense MX quantizer; the grouped MXFP4 quantizer, quantization_impl.py:657-811 with the layout
    of /root/reference/primus_turbo/flydsl/quantization/mxfp4_grouped_quant.py:320-349, is
    ``row_align=1, col_align=256``; ``row_2d`` / ``col_2d``: 32 x 32 blocks counted from the
    group's first row, rows behind the group's end being zeros). Composition of ``mx_quant_rowwise`` / ``mx_quant_colwise`` per group
    (pinned there); the padded placement is pinned by the round trip through ``mx_dequant``
    against the dense quantizer of each group.

    Returns a dict with
      row [Mr, N_pad] codes, row_scale [Mr, N_pad/32]     group g at rows row_offs[g] ...,
                                                          Mr = row_offs[G]; pad rows zero
      col [N, Mc] codes, col_scale [N, Mc/32]             transposed; group g at columns
                                                          col_offs[g] ..., Mc = col_offs[G]
      row_lens / row_offs, col_lens / col_offs            int64 padded lengths and offsets
    (FP4: code arrays packed two per byte along their last axis)."""
    fmt = _fmt(fmt)
    x = np.asarray(x, dtype=F32)
    M, N = x.shape
    gl = np.asarray(group_lens, dtype=np.int64)
    offs = group_offs(gl)
    rl, ro = padded_group_offs(gl, row_align)
    cl, co = padded_group_offs(gl, col_align)
    n_pad = _cdiv(N, 128) * 128
    cpb = 2 if fmt is E2M1 else 1  # codes per byte
    row = np.zeros((int(ro[-1]), n_pad // cpb), dtype=np.uint8)
    row_scale = np.zeros((int(ro[-1]), n_pad // 32), dtype=np.uint8)
    col = np.zeros((N, int(co[-1]) // cpb), dtype=np.uint8)
    col_scale = np.zeros((N, int(co[-1]) // 32), dtype=np.uint8)
    for g in range(len(gl)):
        n = int(gl[g])
        if n == 0:
            continue
        seg = x[offs[g] : offs[g] + n]
        # the pad rows are zero rows of the group: code 0 and scale byte 0 with 1-D blocks, the
        # exponent of their 32 x 32 block with 2-D blocks
        n_r = int(rl[g])
        seg_r = np.zeros((n_r, N), dtype=F32)
        seg_r[:n] = seg
        q, sc = mx_quant_rowwise(seg_r, fmt, use_2d_block=row_2d, use_rht=row_rht)
        row[ro[g] : ro[g] + n_r] = q
        row_scale[ro[g] : ro[g] + n_r] = sc
        q, sc = mx_quant_colwise(seg, fmt, use_2d_block=col_2d, pad=col_align, use_rht=col_rht)
        col[:, co[g] // cpb : co[g + 1] // cpb] = q
        col_scale[:, co[g] // 32 : co[g + 1] // 32] = sc
    return dict(row=row, row_scale=row_scale, col=col, col_scale=col_scale, row_lens=rl, row_offs=ro, col_lens=cl,
                col_offs=co)


def mx_dequant(codes: np.ndarray, scale_bytes: np.ndarray, fmt) -> np.ndarray:
    """float(q) * bits_to_f32(byte << 23) per 32-element block along the last axis
    (/root/reference/csrc/kernels/quantization/dequantization_mxfp8.cu:29-113,
    /root/reference/csrc/kernels/quantization/dequantization_mxfp4.cu:70-160). FP4 input is packed."""
    fmt = _fmt(fmt)
    if fmt is E2M1:
        codes = unpack_fp4(codes)
    v = decode(codes, fmt)
    s = np.repeat(e8m0_to_f32(scale_bytes), 32, axis=-1)[..., : v.shape[-1]]
    with np.errstate(over="ignore", invalid="ignore"):
        return (v * s).astype(F32)
