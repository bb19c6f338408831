"""The reference's own pure-PyTorch CPU formulas, restated (TEST INFRASTRUCTURE ONLY).

Used by ``bench.py`` as the timed CPU baseline and by the tests as a tolerance-level
cross-check. These are the literal formulas of
/root/reference/tests/pytorch/ref/quantization_ref.py:31-68 and
/root/reference/tests/pytorch/ref/gemm_ref.py:13-41, which compute ``x * scale`` in the
input dtype (a 0-dim fp32 scale does not promote a bf16 tensor), i.e. with one more
rounding than the device kernels; on fp32 input they agree with oracle/quantize.py
bit for bit.
"""

from __future__ import annotations

import torch

EPS = 1e-12


def quantize_fp8_tensorwise_ref(x: torch.Tensor, dtype: torch.dtype):
    fp8_max = torch.finfo(dtype).max
    amax = x.abs().amax().to(torch.float32)
    scale = fp8_max / torch.clamp(amax, min=EPS)
    scale_inv = 1.0 / scale
    y = torch.clamp(x * scale, -fp8_max, fp8_max)
    return y.to(dtype), scale.to(torch.float32), scale_inv.to(torch.float32)


def quantize_fp8_rowwise_ref(x: torch.Tensor, dtype: torch.dtype, axis: int):
    axis = axis if axis >= 0 else x.dim() + axis
    fp8_max = torch.finfo(dtype).max
    amax = torch.amax(x.abs(), dim=axis, keepdim=True).to(torch.float32)
    scale = fp8_max / torch.clamp(amax, min=EPS)
    scale_inv = 1.0 / scale
    y = torch.clamp(x * scale, -fp8_max, fp8_max)
    return y.to(dtype), scale.to(torch.float32), scale_inv.to(torch.float32)


def dequantize_fp8_ref(q: torch.Tensor, out_dtype: torch.dtype, scale_inv: torch.Tensor):
    return (q.to(torch.float32) * scale_inv.to(torch.float32)).to(out_dtype)


def gemm_fp8_rowwise_ref(a: torch.Tensor, b: torch.Tensor, dtype=torch.float8_e4m3fn, out_dtype=torch.bfloat16):
    """Rowwise-quantize A [M, K] and B [N, K] along K, then fp32 matmul of the de-quantized
    operands (the accuracy target the north star names for the GEMMs)."""
    aq, _, asi = quantize_fp8_rowwise_ref(a, dtype, -1)
    bq, _, bsi = quantize_fp8_rowwise_ref(b, dtype, -1)
    ad = aq.to(torch.float32) * asi
    bd = bq.to(torch.float32) * bsi
    return (ad @ bd.t()).to(out_dtype)


def quantize_fp8_blockwise_ref(x: torch.Tensor, dtype: torch.dtype, block_m: int, block_n: int):
    """Blockwise quantization of a 2-D tensor with block_m x block_n tiles (1 x 128 for
    activations, 128 x 128 for weights), the formula of the reference's Triton quantizers
    (/root/reference/primus_turbo/triton/quantization/quant_blockwise.py:35-66): scale =
    fp8_max / max(amax, 1e-4), the stored scale is its reciprocal. Returns (codes, scale_inv)
    with scale_inv of shape [ceil(M / block_m), ceil(N / block_n)]."""
    M, N = x.shape
    fp8_max = torch.finfo(dtype).max
    pm, pn = (-M) % block_m, (-N) % block_n
    xp = torch.nn.functional.pad(x.float(), (0, pn, 0, pm))
    t = xp.view((M + pm) // block_m, block_m, (N + pn) // block_n, block_n)
    amax = t.abs().amax(dim=(1, 3), keepdim=True)
    scale = fp8_max / torch.clamp(amax, min=1e-4)
    q = torch.clamp(t * scale, -fp8_max, fp8_max).to(dtype)
    q = q.view(M + pm, N + pn)[:M, :N]
    return q, (1.0 / scale).view((M + pm) // block_m, (N + pn) // block_n)


def gemm_fp8_blockwise_ref(a: torch.Tensor, b: torch.Tensor, dtype=torch.float8_e4m3fn, block: int = 128,
                           out_dtype=torch.bfloat16):
    """DeepSeek-style blockwise GEMM on the CPU: A [M, K] with 1 x block scales, B [N, K] with
    block x block scales, fp32 matmul of the de-quantized operands."""
    aq, asi = quantize_fp8_blockwise_ref(a, dtype, 1, block)
    bq, bsi = quantize_fp8_blockwise_ref(b, dtype, block, block)
    ad = aq.float() * asi.repeat_interleave(block, dim=1)[:, : a.shape[1]]
    bd = bq.float() * bsi.repeat_interleave(block, dim=0)[: b.shape[0]].repeat_interleave(block, dim=1)[:, : b.shape[1]]
    return (ad @ bd.t()).to(out_dtype)


def grouped_gemm_ref(a: torch.Tensor, b: torch.Tensor, seg_lens, trans_b=True):
    out = []
    start = 0
    for i, size in enumerate([int(s) for s in seg_lens]):
        rhs = b[i].t() if trans_b else b[i]
        out.append((a[start : start + size].float() @ rhs.float()).to(a.dtype))
        start += size
    return torch.cat(out)


def grouped_gemm_variable_k_ref(a: torch.Tensor, b: torch.Tensor, seg_lens):
    G = len(seg_lens)
    out = torch.zeros((G, a.shape[1], b.shape[1]), dtype=a.dtype)
    start = 0
    for i, size in enumerate([int(s) for s in seg_lens]):
        out[i] = a[start : start + size].t() @ b[start : start + size]
        start += size
    return out
