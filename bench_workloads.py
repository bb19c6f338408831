"""GEMM workloads of bench.py (the quantizer workload lives in bench.py itself).

Every workload offers: ``step()`` (one pass of the hot path: quantize the bf16 operands and
multiply), ``step_work()`` (flops per step), ``dominant()`` (one launch of the dominant kernel on
pre-quantized operands, for the roofline leg), ``check()`` (parity against the CPU oracle on a
slice) and ``cpu_baseline()`` (the reference's pure-PyTorch formulas on the host cores over a
bounded slice of the same problem).
"""

from __future__ import annotations

import os
import time

import torch

FP8_PEAK_TFLOPS = 5000.0
FP4_PEAK_TFLOPS = 10100.0

# HBM-side bytes per launch of each workload's dominant kernel: rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (KiB per dispatch), each scaled by what the same counter reads for a plain copy of
# 256 MiB launched in the same run (`bench.py --calib-copy`; factors 2.000 and 1.000); the runs are
# summarised under profiles/. (fetched, written) in MiB.
TRAFFIC_MIB = {
    "gemm_fp8_rowwise": (777.2, 151.0),
    "gemm_fp8_blockwise": (349.4, 225.9),
    "gemm_fp8_blockwise_k7168": (696.1, 129.0),
    "gemm_fp8_blockwise_8192": (799.3, 136.3),
    "gemm_mxfp4": (3270.7, 522.8),
    "gemm_mxfp8": (6358.4, 572.4),
    "gemm_mxfp4_n28672": (1434.2, 455.4),
    "gemm_mxfp8_n28672": (2780.0, 448.0),
    # grouped workloads, forward launch: the fetch figure is the average over the forward and dgrad
    # launches of the one kernel symbol that runs both (the counters cannot tell them apart), the
    # write figure is the forward launches' own (they differ from dgrad's by the output width)
    "grouped_gemm_fp8": (4658.7, 256.3),
    "grouped_gemm_fp8_down": (2411.5, 448.8),
    "grouped_gemm_mxfp8": (5354.7, 256.0),
    "grouped_gemm_mxfp8_down": (2650.7, 448.0),
    "grouped_gemm_mxfp4": (2752.2, 256.0),
    "grouped_gemm_mxfp4_down": (1345.3, 448.0),
}


def _traffic(key):
    t = TRAFFIC_MIB.get(key)
    return None if t is None else int((t[0] + t[1]) * 1024 * 1024)


def _randn_bf16(shape, seed, std):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)



def gemm_parity(pairs):
    """(ok, text) for (oracle, result) pairs of output samples: the four figures of the GEMM gate
    (cosine >= 0.9999; max |err| / max |ref| <= 1e-2; |err|_F / |ref|_F <= 1e-2, the relative error of
    the reference's own tests; element-wise |err| <= 2^-7 |ref| + 2^-7 rms(ref row))."""
    from oracle import gemm as OG

    rel = max(OG.max_rel_err(r, g) for r, g in pairs)
    cos = min(OG.cosine(g, r) for r, g in pairs)
    fro = max(OG.rel_fro(r, g) for r, g in pairs)
    exc = max(OG.elementwise_excess(r, g) for r, g in pairs)
    ok = bool(rel <= 1e-2 and cos >= 0.9999 and fro <= 1e-2 and exc <= 1.0)
    return ok, (f"max|err|/max|ref| (relative to the output range)={rel:.2e}, cosine={cos:.6f}, |err|_F/|ref|_F={fro:.2e}, "
                f"element-wise max |err|/(2^-7|ref|+2^-7 rms(row))={exc:.3f}")


class _GemmBase:
    unit = "TFLOP/s"
    dtype = "fp8_e4m3 (fp32 accumulate)"
    bound = "mfma"
    peak = FP8_PEAK_TFLOPS
    metric = "FP8/MXFP4 GEMM TFLOPS & % MFMA peak; quantize GB/s & % HBM peak"

    def step_work(self):
        return 2.0 * self.M * self.N * self.K

    def dominant_work(self):
        return 2.0 * self.M * self.N * self.K


class GemmFp8Rowwise(_GemmBase):
    """BASELINE config 1: E4M3 rowwise-scaled NT GEMM, A and B 8192x8192 bf16 ~N(0, 0.02)."""

    name = "fp8_e4m3_rowwise_gemm_8192x8192x8192_bf16_out (quantize A, quantize B, multiply)"
    dominant_name = "gemm_fp8_nt_kernel<256x256 tile, per-row/per-column scales>"

    def __init__(self, dev, M=8192, N=8192, K=8192):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.core.low_precision import (
            Float8QuantConfig,
            Format,
            ScalingGranularity,
        )
        from primus_turbo.pytorch.kernels.gemm.gemm_fp8_impl import gemm_fp8_impl

        self.turbo, self.G = turbo, ScalingGranularity
        self.M, self.N, self.K = M, N, K
        self.cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.ROWWISE)
        self.a_cpu = _randn_bf16((M, K), 1, 0.02)
        self.b_cpu = _randn_bf16((N, K), 2, 0.02)
        self.a, self.b = self.a_cpu.to(dev), self.b_cpu.to(dev)
        self._impl = gemm_fp8_impl
        # pre-quantized operands for the dominant-kernel leg
        self.aq, self.as_inv = turbo.ops.quantize_fp8(self.a, turbo.float8_e4m3, ScalingGranularity.ROWWISE, axis=-1)
        self.bq, self.bs_inv = turbo.ops.quantize_fp8(self.b, turbo.float8_e4m3, ScalingGranularity.ROWWISE, axis=-1)
        self.out = None

    def step(self):
        self.out = self.turbo.ops.gemm_fp8(self.a, self.b, trans_a=False, trans_b=True, out_dtype=torch.bfloat16, config=self.cfg)
        return self.out

    def dominant(self):
        return self._impl(self.aq, self.as_inv, False, self.bq, self.bs_inv, True, torch.bfloat16, False, self.G.ROWWISE.value, 0)

    def check(self):
        """Rows [0, 64) and [M-64, M) of the product against the oracle (fp32 matmul of the
        dequantized operands); quantized bytes of those rows bit-exact."""
        import numpy as np

        from oracle import gemm as OG
        from oracle import quantize as Q

        out = self.step().float().cpu().numpy()
        rows = np.r_[0:64, self.M - 64 : self.M]
        a = self.a_cpu.float().numpy()[rows]
        b = self.b_cpu.float().numpy()
        aq, asi = Q.fp8_rowwise(a, -1, "e4m3")
        bq, bsi = Q.fp8_rowwise(b, -1, "e4m3")
        same = np.array_equal(self.aq.cpu().view(torch.uint8).numpy()[rows], aq)
        same = same and np.array_equal(np.ascontiguousarray(self.as_inv.cpu().numpy()[rows]).view(np.int32), np.ascontiguousarray(asi).view(np.int32))
        same = same and np.array_equal(self.bq.cpu().view(torch.uint8).numpy(), bq)
        ref = OG.gemm_dequantized(Q.fp8_dequant(aq, asi, "e4m3"), Q.fp8_dequant(bq, bsi, "e4m3"), trans_b=True)
        # the product is rounded to bf16: compare against the bf16-rounded oracle
        ref_t = torch.from_numpy(np.ascontiguousarray(ref, dtype=np.float32)).to(torch.bfloat16).float().numpy()
        ok, text = gemm_parity([(ref_t, out[rows])])
        return bool(same and ok), f"quantized bytes and activation scales bit-exact: {same}; 128 output rows vs oracle: {text}"

    def cpu_baseline(self):
        """The reference's CPU formulas on an M-slice: rowwise quantize of the slice and of all of
        B, dequantize, fp32 matmul. Scaled to the metric's unit (flops of the slice / time)."""
        from oracle import cpu_reference as R

        rows = self.M  # the whole problem: a few seconds on 16 cores
        a = self.a_cpu[:rows]
        b = self.b_cpu
        t0 = time.perf_counter()
        aq, _, asi = R.quantize_fp8_rowwise_ref(a, torch.float8_e4m3fn, axis=-1)
        bq, _, bsi = R.quantize_fp8_rowwise_ref(b, torch.float8_e4m3fn, axis=-1)
        y = (aq.float() * asi) @ (bq.float() * bsi).t()
        y = y.to(torch.bfloat16)
        dt = time.perf_counter() - t0
        return dict(
            value=round(2.0 * rows * self.N * self.K / dt / 1e12, 4),
            unit="TFLOP/s",
            cores=torch.get_num_threads(),
            kind="port",
            sample=f"first {rows} rows of A against all of B (quantize both, dequantize, fp32 matmul), "
            f"{dt:.1f} s, {os.cpu_count()} logical CPUs visible",
        )


class GemmFp8Blockwise(_GemmBase):
    """BASELINE config 2: DeepSeek-style blockwise GEMM, activations 1x128, weights 128x128."""

    dominant_name = "gemm_fp8_block8_kernel<256x256 tile, eight wavefronts, 1x128 * 128x128 block scales>"

    def __init__(self, dev, M=16384, N=7168, K=2048):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.core.low_precision import (
            Float8QuantConfig,
            Format,
            ScalingGranularity,
        )
        from primus_turbo.pytorch.kernels.gemm.gemm_fp8_impl import gemm_fp8_impl
        from primus_turbo.pytorch.kernels.quantization.quantization_impl import (
            quant_fp8_blockwise_for_weight_impl,
            quant_fp8_blockwise_kmajor_impl,
        )

        self.turbo, self.G = turbo, ScalingGranularity
        self.M, self.N, self.K = M, N, K
        self.name = f"fp8_e4m3_blockwise_gemm_{M}x{N}x{K}_bf16_out (1x128 activations, 128x128 weights)"
        self.cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.BLOCKWISE, block_size=128)
        self.a_cpu = _randn_bf16((M, K), 3, 1.0)
        self.b_cpu = _randn_bf16((N, K), 4, 1.0)
        self.a, self.b = self.a_cpu.to(dev), self.b_cpu.to(dev)
        self._impl = gemm_fp8_impl
        # the operands as the op's forward hands them to the kernel: row scales of A block-major
        self.aq, as_kmajor, _, _ = quant_fp8_blockwise_kmajor_impl(self.a, turbo.float8_e4m3, 128, False)
        self.as_inv = as_kmajor.t()
        self.bq, self.bs_inv = quant_fp8_blockwise_for_weight_impl(self.b, turbo.float8_e4m3, 128)

    def step(self):
        return self.turbo.ops.gemm_fp8(self.a, self.b, trans_a=False, trans_b=True, out_dtype=torch.bfloat16, config=self.cfg)

    def dominant(self):
        return self._impl(self.aq, self.as_inv, False, self.bq, self.bs_inv, True, torch.bfloat16, False, self.G.BLOCKWISE.value, 0)

    def check(self):
        import numpy as np

        from oracle import gemm as OG
        from oracle import quantize as Q

        out = self.step().float().cpu().numpy()
        rows = np.r_[0:64, self.M - 64 : self.M]
        a = self.a_cpu.float().numpy()[rows]
        b = self.b_cpu.float().numpy()
        aq, asi = Q.fp8_blockwise(a, 1, "e4m3", 128)
        bq, bsi = Q.fp8_blockwise_weight(b, "e4m3", 128)
        same = np.array_equal(self.aq.cpu().view(torch.uint8).numpy()[rows], aq)
        same = same and np.array_equal(self.bq.cpu().view(torch.uint8).numpy(), bq)
        ref = OG.gemm_dequantized(
            Q.fp8_blockwise_dequant(aq, asi, 1, "e4m3", 128), Q.fp8_blockwise_weight_dequant(bq, bsi, "e4m3", 128), trans_b=True
        )
        ref_t = torch.from_numpy(np.ascontiguousarray(ref, dtype=np.float32)).to(torch.bfloat16).float().numpy()
        ok, text = gemm_parity([(ref_t, out[rows])])
        return bool(same and ok), f"quantized bytes bit-exact: {same}; 128 output rows vs oracle: {text}"

    def cpu_baseline(self):
        from oracle import cpu_reference as R

        rows = self.M
        a = self.a_cpu[:rows]
        b = self.b_cpu
        t0 = time.perf_counter()
        y = R.gemm_fp8_blockwise_ref(a, b, torch.float8_e4m3fn, 128)
        dt = time.perf_counter() - t0
        del y
        return dict(
            value=round(2.0 * rows * self.N * self.K / dt / 1e12, 4),
            unit="TFLOP/s",
            cores=torch.get_num_threads(),
            kind="port",
            sample=f"first {rows} rows of A against all of B (blockwise quantize, dequantize, fp32 matmul), "
            f"{dt:.1f} s, {os.cpu_count()} logical CPUs visible",
        )


class GemmMx(_GemmBase):
    """BASELINE config 4: MX-scaled GEMM (E8M0 scale per 32 elements of K, applied by the matrix
    core): MXFP4 (E2M1) or its MXFP8 (E4M3) fallback, bf16 source ~N(0, 1), bf16 output."""

    def __init__(self, dev, fp4=True, M=16384, N=16384, K=16384):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.core.low_precision import (
            Float4QuantConfig,
            Float8QuantConfig,
            Format,
            ScaleDtype,
            ScalingGranularity,
            ScalingRecipe,
        )
        from primus_turbo.pytorch.kernels.gemm import gemm_fp4_impl, gemm_fp8_impl
        from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

        self.turbo, self.G, self.fp4 = turbo, ScalingGranularity, fp4
        self.M, self.N, self.K = M, N, K
        kind = "mxfp4_e2m1" if fp4 else "mxfp8_e4m3"
        self.name = f"{kind}_gemm_{M}x{N}x{K}_bf16_out (quantize A 1x32, quantize B 32x32, multiply)"
        self.dtype = ("fp4_e2m1" if fp4 else "fp8_e4m3") + " with E8M0 block scales (fp32 accumulate)"
        self.peak = FP4_PEAK_TFLOPS if fp4 else FP8_PEAK_TFLOPS
        self.dominant_name = "gemm_fp8_nt_kernel<256x256 tile, E8M0 block scales in the MFMA>"
        self.fmt = "e2m1" if fp4 else "e4m3"
        if fp4:
            self.cfg = Float4QuantConfig()
            self.qdt = torch.float4_e2m1fn_x2
            self._quant, self._impl = qi.quantize_mxfp4_impl, gemm_fp4_impl.gemm_fp4_impl
        else:
            self.cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE,
                                         block_size=32, scale_dtype=ScaleDtype.E8M0)
            self.qdt = torch.float8_e4m3fn
            self._quant, self._impl = qi.quantize_mxfp8_impl, gemm_fp8_impl.gemm_fp8_impl
        self.a_cpu = _randn_bf16((M, K), 5, 1.0)
        self.b_cpu = _randn_bf16((N, K), 6, 1.0)
        self.a, self.b = self.a_cpu.to(dev), self.b_cpu.to(dev)
        self.aq, self.as_ = self._quant(self.a, self.qdt, 1, 32)
        self.bq, self.bs = self._quant(self.b, self.qdt, 1, 32, scaling_recipe=ScalingRecipe(use_2d_block=True))

    def step(self):
        op = self.turbo.ops.gemm_fp4 if self.fp4 else self.turbo.ops.gemm_fp8
        return op(self.a, self.b, trans_a=False, trans_b=True, out_dtype=torch.bfloat16, config=self.cfg)

    def dominant(self):
        return self._impl(self.aq, self.as_, False, self.bq, self.bs, True, torch.bfloat16, False,
                          self.G.MX_BLOCKWISE.value, 0)

    def check(self):
        """Quantized codes and E8M0 bytes of 128 rows of A and the first 128 rows of B bit-exact
        with the oracle; the product of those A rows against the oracle's de-quantized matmul."""
        import numpy as np

        from oracle import gemm as OG
        from oracle import quantize as Q

        def u8(t):
            return t.contiguous().view(torch.uint8).cpu().numpy()

        out = self.dominant().float().cpu().numpy()
        rows = np.r_[0:64, self.M - 64 : self.M]
        a = self.a_cpu.float().numpy()[rows]
        aq, asc = Q.mx_quant_rowwise(a, self.fmt)
        bq, bsc = Q.mx_quant_rowwise(self.b_cpu.float().numpy()[:128], self.fmt, use_2d_block=True)
        kb = self.K // 32
        same = np.array_equal(u8(self.aq)[rows], aq) and np.array_equal(u8(self.as_)[rows][:, :kb], asc[:, :kb])
        same = same and np.array_equal(u8(self.bq)[:128], bq) and np.array_equal(u8(self.bs)[:128, :kb], bsc[:, :kb])
        nb = min(self.N, 2048)  # output columns checked
        b_deq = Q.mx_dequant(u8(self.bq)[:nb], u8(self.bs)[:nb], self.fmt)
        ref = OG.gemm_dequantized(Q.mx_dequant(aq, asc, self.fmt), b_deq, trans_b=True)
        ref_t = torch.from_numpy(np.ascontiguousarray(ref, dtype=np.float32)).to(torch.bfloat16).float().numpy()
        ok, text = gemm_parity([(ref_t, out[rows][:, :nb])])
        return bool(same and ok), f"codes and E8M0 bytes bit-exact: {same}; 128 x 2048 outputs vs oracle: {text}"

    def cpu_baseline(self):
        """The oracle (numpy restatement of the reference's MX quantizer) plus an fp32 matmul on a
        slice: 256 rows of A against 2048 rows of B."""
        import numpy as np

        from oracle import quantize as Q

        ra, rb = 256, 2048
        a = self.a_cpu[:ra].float().numpy()
        b = self.b_cpu[:rb].float().numpy()
        t0 = time.perf_counter()
        aq, asc = Q.mx_quant_rowwise(a, self.fmt)
        bq, bsc = Q.mx_quant_rowwise(b, self.fmt, use_2d_block=True)
        y = Q.mx_dequant(aq, asc, self.fmt) @ Q.mx_dequant(bq, bsc, self.fmt).T
        dt = time.perf_counter() - t0
        del y
        return dict(
            value=round(2.0 * ra * rb * self.K / dt / 1e12, 5),
            unit="TFLOP/s",
            cores=torch.get_num_threads(),
            kind="port",
            sample=f"{ra} rows of A against {rb} rows of B (MX quantize both, dequantize, fp32 matmul), {dt:.1f} s, "
            f"{os.cpu_count()} logical CPUs visible",
        )


def _zipf_group_lens(groups, total, seed):
    """Per-expert token counts ~ Zipf(1.2) over a random expert order, two experts empty."""
    import numpy as np

    rng = np.random.default_rng(seed)
    w = rng.permutation((1.0 + np.arange(groups)) ** -1.2)
    w[rng.choice(groups, 2, replace=False)] = 0
    lens = np.floor(w / w.sum() * total).astype(np.int64)
    lens[np.argmax(lens)] += total - lens.sum()
    return lens


class GroupedGemmFp8(_GemmBase):
    """BASELINE config 3: MoE grouped GEMM of one GPU's experts (32 experts, 32768 routed tokens,
    Zipf(1.2) counts with empty experts), blockwise 128 scales; a step is forward + dgrad + wgrad
    of one expert layer through the autograd op."""

    dominant_name = "gemm_fp8_block8_kernel<256x256 tile, eight wavefronts, row groups, 1x128 * 128x128 block scales> (forward)"

    def __init__(self, dev, N=4096, K=7168, groups=32, tokens=32768):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, Format, ScalingGranularity
        from primus_turbo.pytorch.kernels.grouped_gemm import grouped_gemm_fp8_impl as gg
        from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

        self.turbo, self.G, self.gg, self.qi = turbo, ScalingGranularity, gg, qi
        self.M, self.N, self.K, self.groups = tokens, N, K, groups
        self.name = (f"moe_grouped_gemm_fp8_blockwise_{groups}experts_{tokens}tokens_zipf1.2_k{K}_n{N} "
                     "(forward + dgrad + wgrad, quantizers included)")
        self.cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.BLOCKWISE, block_size=128)
        self.lens = _zipf_group_lens(groups, tokens, 7)
        self.gl = torch.from_numpy(self.lens).to(dev)
        self.offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(self.gl)
        self.x_cpu = _randn_bf16((tokens, K), 7, 1.0)
        self.w_cpu = _randn_bf16((groups, N, K), 8, 1.0)
        self.x = self.x_cpu.to(dev).requires_grad_(True)
        self.w = self.w_cpu.to(dev).requires_grad_(True)
        self.dy = _randn_bf16((tokens, N), 9, 1.0).to(dev)
        self.qr, _, self.sr, _, _, _ = qi.quant_fp8_blockwise_segment_m_row_col_impl(
            self.x.detach(), torch.float8_e4m3fn, 128, self.gl, self.offs, N)
        self.wq, self.ws = qi.quant_fp8_blockwise_for_weight_impl(self.w.detach(), torch.float8_e4m3fn, 128)

    def step_work(self):
        return 3 * 2.0 * self.M * self.N * self.K

    def step(self):
        self.x.grad = None
        self.w.grad = None
        y = self.turbo.ops.grouped_gemm_fp8(self.x, self.w, self.gl, self.offs, trans_b=True, config=self.cfg)
        y.backward(self.dy)
        return y

    def dominant(self):
        return self.gg.grouped_gemm_fp8_impl(self.qr, self.wq, self.sr, self.ws, self.gl, self.offs, False, True,
                                             torch.bfloat16, self.G.BLOCKWISE.value, None, 0)

    def kernels(self):
        """The three GEMM launches of the step on pre-quantized operands, as the autograd function
        issues them: (name, callable, flops)."""
        qi, gg, gran = self.qi, self.gg, self.G.BLOCKWISE.value
        f8 = torch.float8_e4m3fn
        if not hasattr(self, "_bwd"):
            x_row, x_col_t, x_srow, x_scol, _, _ = qi.quant_fp8_blockwise_segment_m_row_col_t_impl(
                self.x.detach(), f8, 128, self.gl, self.offs)
            g_row, g_col_t, g_srow, g_scol, vk_lens, vk_offs = qi.quant_fp8_blockwise_segment_m_row_col_t_impl(
                self.dy, f8, 128, self.gl, self.offs)
            wq, wq_t, ws = qi.quant_fp8_blockwise_for_weight_dual_impl(self.w.detach(), f8, block_size=128)
            ws_t = ws.transpose(-2, -1).contiguous()
            self._bwd = (x_col_t, x_scol, g_row, g_srow, g_col_t, g_scol, vk_lens, vk_offs, wq_t, ws_t)
        x_col_t, x_scol, g_row, g_srow, g_col_t, g_scol, vk_lens, vk_offs, wq_t, ws_t = self._bwd
        flops = 2.0 * self.M * self.N * self.K

        def dgrad():
            return gg.grouped_gemm_fp8_impl(g_row, wq_t, g_srow, ws_t, self.gl, self.offs, False, True, torch.bfloat16,
                                            gran, None, 0)

        def wgrad():
            return gg.grouped_gemm_fp8_variable_k_impl(x_col_t, g_col_t, x_scol, g_scol, vk_lens, vk_offs, False, True,
                                                       True, torch.bfloat16, gran, None, 0)

        return [("forward", self.dominant, flops), ("dgrad", dgrad, flops), ("wgrad_variable_k", wgrad, flops)]

    def check(self):
        """Forward rows of the first and of the last non-empty expert (up to 64 each) against the
        oracle's de-quantized matmul; their quantized bytes bit-exact."""
        import numpy as np

        from oracle import gemm as OG
        from oracle import quantize as Q

        out = self.dominant().float().cpu().numpy()
        offs = np.concatenate([[0], np.cumsum(self.lens)])
        live = [g for g in range(self.groups) if self.lens[g] > 0]
        same, pairs = True, []
        for g in (live[0], live[-1]):
            r0, r1 = int(offs[g]), int(min(offs[g] + 64, offs[g + 1]))
            aq, asi = Q.fp8_blockwise(self.x_cpu.float().numpy()[r0:r1], 1, "e4m3", 128)
            bq, bsi = Q.fp8_blockwise_weight(self.w_cpu[g].float().numpy(), "e4m3", 128)
            same = same and np.array_equal(self.qr[r0:r1].view(torch.uint8).cpu().numpy(), aq)
            same = same and np.array_equal(self.wq[g].view(torch.uint8).cpu().numpy(), bq)
            ref = OG.gemm_dequantized(Q.fp8_blockwise_dequant(aq, asi, 1, "e4m3", 128),
                                      Q.fp8_blockwise_weight_dequant(bq, bsi, "e4m3", 128), trans_b=True)
            ref_t = torch.from_numpy(np.ascontiguousarray(ref, dtype=np.float32)).to(torch.bfloat16).float().numpy()
            pairs.append((ref_t, out[r0:r1]))
        ok, text = gemm_parity(pairs)
        return bool(same and ok), f"quantized bytes bit-exact: {same}; rows of two experts vs oracle: {text}"

    def cpu_baseline(self):
        """The reference's CPU formulas (blockwise quantize, dequantize, per-expert fp32 matmul) for
        the forward product of the four experts with the most tokens."""
        from oracle import cpu_reference as R

        import numpy as np

        offs = np.concatenate([[0], np.cumsum(self.lens)])
        top = np.argsort(-self.lens)[:4]
        rows = int(self.lens[top].sum())
        t0 = time.perf_counter()
        for g in top:
            y = R.gemm_fp8_blockwise_ref(self.x_cpu[int(offs[g]) : int(offs[g + 1])], self.w_cpu[g], torch.float8_e4m3fn, 128)
        dt = time.perf_counter() - t0
        del y
        return dict(
            value=round(2.0 * rows * self.N * self.K / dt / 1e12, 4),
            unit="TFLOP/s",
            cores=torch.get_num_threads(),
            kind="port",
            sample=f"forward product of the 4 largest experts ({rows} of {self.M} tokens: blockwise quantize, "
            f"dequantize, fp32 matmul), {dt:.1f} s, {os.cpu_count()} logical CPUs visible",
        )


class GroupedGemmMxfp8(_GemmBase):
    """The MoE configuration (32 experts, 32768 routed tokens, Zipf(1.2) counts with empty experts)
    through the grouped MXFP8 path: grouped MX quantizers (rows padded to 32 per expert, transposed
    columns to 128), forward + dgrad row-group GEMMs and the variable-K wgrad GEMM."""

    dominant_name = "gemm_fp8_nt_kernel<256x256 tile, row groups, E8M0 block scales in the MFMA> (forward)"
    dtype = "fp8_e4m3 with E8M0 block scales (fp32 accumulate)"

    def __init__(self, dev, N=4096, K=7168, groups=32, tokens=32768):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.core.low_precision import Float8QuantConfig, Format, ScaleDtype, ScalingGranularity, ScalingRecipe
        from primus_turbo.pytorch.kernels.grouped_gemm import grouped_gemm_fp8_impl as gg
        from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

        self.turbo, self.G, self.gg, self.qi = turbo, ScalingGranularity, gg, qi
        self.M, self.N, self.K, self.groups = tokens, N, K, groups
        self.name = (f"moe_grouped_gemm_mxfp8_{groups}experts_{tokens}tokens_zipf1.2_k{K}_n{N} "
                     "(forward + dgrad + wgrad, quantizers included)")
        self.cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.MX_BLOCKWISE, block_size=32,
                                     scale_dtype=ScaleDtype.E8M0)
        self.lens = _zipf_group_lens(groups, tokens, 7)
        self.gl = torch.from_numpy(self.lens).to(dev)
        self.offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(self.gl)
        self.x_cpu = _randn_bf16((tokens, K), 7, 1.0)
        self.w_cpu = _randn_bf16((groups, N, K), 8, 1.0)
        self.x = self.x_cpu.to(dev).requires_grad_(True)
        self.w = self.w_cpu.to(dev).requires_grad_(True)
        self.dy = _randn_bf16((tokens, N), 9, 1.0).to(dev)
        self.qr, self.sr, _, self.offs_row = qi.grouped_quantize_mxfp8_impl(self.x.detach(), torch.float8_e4m3fn, 1, 32,
                                                                            self.gl, self.offs)
        self.wq, self.ws = qi.quantize_mxfp8_impl(self.w.detach(), torch.float8_e4m3fn, 2, 32,
                                                  scaling_recipe=ScalingRecipe(use_2d_block=True))
        self.fmt = "e4m3"

    def step_work(self):
        return 3 * 2.0 * self.M * self.N * self.K

    def step(self):
        self.x.grad = None
        self.w.grad = None
        y = self.turbo.ops.grouped_gemm_fp8(self.x, self.w, self.gl, self.offs, trans_b=True, config=self.cfg)
        y.backward(self.dy)
        return y

    def dominant(self):
        return self.gg.grouped_gemm_fp8_impl(self.qr, self.wq, self.sr, self.ws, self.gl, self.offs_row, False, True,
                                             torch.bfloat16, self.G.MX_BLOCKWISE.value, None, 0, False, self.offs)

    def _backward_operands(self):
        """(grad row codes / scales, grad column codes / scales, activation column codes / scales,
        transposed weight codes / scales, padded row offsets, padded column lens / offsets) as
        the autograd function prepares them."""
        from primus_turbo.pytorch.core.low_precision import ScalingRecipe

        qi, f8 = self.qi, torch.float8_e4m3fn
        _, _, a_col, a_col_s, _, _, _, _ = qi.grouped_quantize_mxfp8_impl(self.x.detach(), f8, None, 32, self.gl, self.offs,
                                                                          with_trans=True)
        g_row, g_row_s, g_col, g_col_s, _, offs_row, lens_col, offs_col = qi.grouped_quantize_mxfp8_impl(
            self.dy, f8, None, 32, self.gl, self.offs, with_trans=True)
        r2 = ScalingRecipe(use_2d_block=True)
        _, _, b_col, b_col_s = qi.quantize_mxfp8_impl(self.w.detach(), f8, None, 32, with_trans=True, scaling_recipe=r2,
                                                      scaling_recipe_for_trans=r2)
        return g_row, g_row_s, g_col, g_col_s, a_col, a_col_s, b_col, b_col_s, offs_row, lens_col, offs_col

    def _impls(self):
        return self.gg.grouped_gemm_fp8_impl, self.gg.grouped_gemm_fp8_variable_k_impl

    def kernels(self):
        """The three GEMM launches of the step on pre-quantized operands, as the autograd function
        issues them: (name, callable, flops)."""
        if not hasattr(self, "_bwd"):
            self._bwd = self._backward_operands()
        g_row, g_row_s, g_col, g_col_s, a_col, a_col_s, b_col, b_col_s, offs_row, lens_col, offs_col = self._bwd
        rows_impl, vk_impl = self._impls()
        gran, flops = self.G.MX_BLOCKWISE.value, 2.0 * self.M * self.N * self.K

        def dgrad():
            return rows_impl(g_row, b_col, g_row_s, b_col_s, self.gl, offs_row, False, True, torch.bfloat16, gran, None, 0,
                             False, self.offs)

        def wgrad():
            return vk_impl(g_col, a_col, g_col_s, a_col_s, lens_col, offs_col, False, False, False, torch.bfloat16, gran,
                           None, 0)

        return [("forward", self.dominant, flops), ("dgrad", dgrad, flops), ("wgrad_variable_k", wgrad, flops)]

    def check(self):
        """Forward rows of the first and of the last non-empty expert (up to 64 each) against the
        oracle's de-quantized matmul; their codes and E8M0 bytes bit-exact."""
        import numpy as np

        from oracle import gemm as OG
        from oracle import quantize as Q

        def u8(t):
            return t.contiguous().view(torch.uint8).cpu().numpy()

        out = self.dominant().float().cpu().numpy()
        offs = np.concatenate([[0], np.cumsum(self.lens)])
        orow = self.offs_row.cpu().numpy()
        live = [g for g in range(self.groups) if self.lens[g] > 0]
        same, pairs = True, []
        for g in (live[0], live[-1]):
            n = int(min(64, self.lens[g]))
            r0, p0 = int(offs[g]), int(orow[g])
            aq, asc = Q.mx_quant_rowwise(self.x_cpu.float().numpy()[r0 : r0 + n], self.fmt)
            same = same and np.array_equal(u8(self.qr)[p0 : p0 + n], aq) and np.array_equal(u8(self.sr)[p0 : p0 + n], asc)
            w_deq = Q.mx_dequant(u8(self.wq[g]), u8(self.ws[g]), self.fmt)
            ref = OG.gemm_dequantized(Q.mx_dequant(aq, asc, self.fmt), w_deq, trans_b=True)
            ref_t = torch.from_numpy(np.ascontiguousarray(ref, dtype=np.float32)).to(torch.bfloat16).float().numpy()
            pairs.append((ref_t, out[r0 : r0 + n]))
        ok, text = gemm_parity(pairs)
        return bool(same and ok), f"codes and E8M0 bytes bit-exact: {same}; rows of two experts vs oracle: {text}"

    def cpu_baseline(self):
        """The numpy oracle (MX quantize, de-quantize) plus an fp32 matmul for 256 tokens of the
        largest expert against 2048 of its output features."""
        import numpy as np

        from oracle import quantize as Q

        g = int(np.argmax(self.lens))
        r0 = int(np.concatenate([[0], np.cumsum(self.lens)])[g])
        a = self.x_cpu[r0 : r0 + 256].float().numpy()
        b = self.w_cpu[g, :2048].float().numpy()
        t0 = time.perf_counter()
        aq, asc = Q.mx_quant_rowwise(a, self.fmt)
        bq, bsc = Q.mx_quant_rowwise(b, self.fmt, use_2d_block=True)
        y = Q.mx_dequant(aq, asc, self.fmt) @ Q.mx_dequant(bq, bsc, self.fmt).T
        dt = time.perf_counter() - t0
        del y
        return dict(value=round(2.0 * 256 * 2048 * self.K / dt / 1e12, 5), unit="TFLOP/s", cores=torch.get_num_threads(),
                    kind="port", sample=f"256 tokens of the largest expert against 2048 output features (MX quantize both, "
                    f"dequantize, fp32 matmul), {dt:.1f} s, {os.cpu_count()} logical CPUs visible")


class GroupedGemmMxfp4(GroupedGemmMxfp8):
    """The same MoE configuration through the grouped MXFP4 path: rows quantized in place,
    transposed columns padded to 256 tokens per expert, packed E2M1 operands."""

    dominant_name = "gemm_fp8_nt_kernel<256x256 tile, row groups, MXFP4 operands, E8M0 block scales in the MFMA> (forward)"
    dtype = "fp4_e2m1 with E8M0 block scales (fp32 accumulate)"
    peak = FP4_PEAK_TFLOPS

    def __init__(self, dev, N=4096, K=7168, groups=32, tokens=32768):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.core.low_precision import Float4QuantConfig, ScalingGranularity, ScalingRecipe, float4_e2m1fn_x2
        from primus_turbo.pytorch.kernels.grouped_gemm import grouped_gemm_fp4_impl as gg
        from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

        self.turbo, self.G, self.gg, self.qi = turbo, ScalingGranularity, gg, qi
        self.M, self.N, self.K, self.groups = tokens, N, K, groups
        self.name = (f"moe_grouped_gemm_mxfp4_{groups}experts_{tokens}tokens_zipf1.2_k{K}_n{N} "
                     "(forward + dgrad + wgrad, quantizers included)")
        self.cfg = Float4QuantConfig()
        self.lens = _zipf_group_lens(groups, tokens, 7)
        self.gl = torch.from_numpy(self.lens).to(dev)
        self.offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(self.gl)
        self.x_cpu = _randn_bf16((tokens, K), 7, 1.0)
        self.w_cpu = _randn_bf16((groups, N, K), 8, 1.0)
        self.x = self.x_cpu.to(dev).requires_grad_(True)
        self.w = self.w_cpu.to(dev).requires_grad_(True)
        self.dy = _randn_bf16((tokens, N), 9, 1.0).to(dev)
        self.qr, self.sr, _, self.offs_row = qi.grouped_quantize_mxfp4_impl(self.x.detach(), float4_e2m1fn_x2, 1, 32,
                                                                            self.gl, self.offs)
        self.wq, self.ws = qi.quantize_mxfp4_impl(self.w.detach(), float4_e2m1fn_x2, 2, 32,
                                                  scaling_recipe=ScalingRecipe(use_2d_block=True))
        self.fmt = "e2m1"

    def step(self):
        self.x.grad = None
        self.w.grad = None
        y = self.turbo.ops.grouped_gemm_fp4(self.x, self.w, self.gl, self.offs, trans_b=True, config=self.cfg)
        y.backward(self.dy)
        return y

    def dominant(self):
        return self.gg.grouped_gemm_fp4_impl(self.qr, self.wq, self.sr, self.ws, self.gl, self.offs_row, False, True,
                                             torch.bfloat16, self.G.MX_BLOCKWISE.value, None, 0, False, self.offs)

    def _backward_operands(self):
        from primus_turbo.pytorch.core.low_precision import ScalingRecipe, float4_e2m1fn_x2 as f4

        qi = self.qi
        plain, rht = ScalingRecipe(), ScalingRecipe(use_rht=True)
        _, _, a_col, a_col_s, _, _, _, _ = qi.grouped_quantize_mxfp4_impl(self.x.detach(), f4, None, 32, self.gl, self.offs,
                                                                          with_trans=True, scaling_recipe=plain,
                                                                          scaling_recipe_for_trans=rht)
        g_row, g_row_s, g_col, g_col_s, _, _, lens_col, offs_col = qi.grouped_quantize_mxfp4_impl(
            self.dy, f4, None, 32, self.gl, self.offs, with_trans=True, scaling_recipe=plain, scaling_recipe_for_trans=rht)
        r2 = ScalingRecipe(use_2d_block=True)
        _, _, b_col, b_col_s = qi.quantize_mxfp4_impl(self.w.detach(), f4, None, 32, with_trans=True, scaling_recipe=r2,
                                                      scaling_recipe_for_trans=r2)
        return g_row, g_row_s, g_col, g_col_s, a_col, a_col_s, b_col, b_col_s, self.offs, lens_col, offs_col

    def _impls(self):
        return self.gg.grouped_gemm_fp4_impl, self.gg.grouped_gemm_fp4_variable_k_impl


def _keyed(key, make):
    def build(dev):
        wl = make(dev)
        wl.traffic = _traffic(key)
        return wl

    return build


def register(workloads):
    workloads["gemm_fp8_rowwise"] = GemmFp8Rowwise
    workloads["gemm_fp8_blockwise"] = GemmFp8Blockwise
    workloads["gemm_fp8_blockwise_k7168"] = lambda dev: GemmFp8Blockwise(dev, 16384, 4096, 7168)
    workloads["gemm_fp8_blockwise_8192"] = lambda dev: GemmFp8Blockwise(dev, 8192, 8192, 8192)
    workloads["gemm_mxfp4"] = lambda dev: GemmMx(dev, True, 16384, 16384, 16384)
    workloads["gemm_mxfp4_n28672"] = lambda dev: GemmMx(dev, True, 8192, 28672, 8192)
    workloads["gemm_mxfp8"] = lambda dev: GemmMx(dev, False, 16384, 16384, 16384)
    workloads["gemm_mxfp8_n28672"] = lambda dev: GemmMx(dev, False, 8192, 28672, 8192)
    workloads["grouped_gemm_fp8"] = lambda dev: GroupedGemmFp8(dev, 4096, 7168)
    workloads["grouped_gemm_fp8_down"] = lambda dev: GroupedGemmFp8(dev, 7168, 2048)
    workloads["grouped_gemm_mxfp8"] = lambda dev: GroupedGemmMxfp8(dev, 4096, 7168)
    workloads["grouped_gemm_mxfp8_down"] = lambda dev: GroupedGemmMxfp8(dev, 7168, 2048)
    workloads["grouped_gemm_mxfp4"] = lambda dev: GroupedGemmMxfp4(dev, 4096, 7168)
    workloads["grouped_gemm_mxfp4_down"] = lambda dev: GroupedGemmMxfp4(dev, 7168, 2048)
    for key in list(workloads):
        if key in TRAFFIC_MIB:
            workloads[key] = _keyed(key, workloads[key])
