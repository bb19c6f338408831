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


def _randn_bf16(shape, seed, std):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)


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
        same = same and np.array_equal(self.bq.cpu().view(torch.uint8).numpy(), bq)
        ref = OG.gemm_dequantized(Q.fp8_dequant(aq, asi, "e4m3"), Q.fp8_dequant(bq, bsi, "e4m3"), trans_b=True)
        # the product is rounded to bf16: compare against the bf16-rounded oracle
        ref_t = torch.from_numpy(np.ascontiguousarray(ref, dtype=np.float32)).to(torch.bfloat16).float().numpy()
        rel = OG.max_rel_err(ref_t, out[rows])
        cos = OG.cosine(out[rows], ref_t)
        ok = bool(same and rel <= 1e-2 and cos >= 0.9999)
        return ok, f"quantized bytes bit-exact; 128 output rows vs oracle: max_rel_err={rel:.2e}, cosine={cos:.6f}"

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

    dominant_name = "gemm_fp8_nt_kernel<128x128 tile, 1x128 * 128x128 block scales>"

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
            quant_fp8_blockwise_impl,
        )

        self.turbo, self.G = turbo, ScalingGranularity
        self.M, self.N, self.K = M, N, K
        self.name = f"fp8_e4m3_blockwise_gemm_{M}x{N}x{K}_bf16_out (1x128 activations, 128x128 weights)"
        self.cfg = Float8QuantConfig(format=Format.E4M3, granularity=ScalingGranularity.BLOCKWISE, block_size=128)
        self.a_cpu = _randn_bf16((M, K), 3, 1.0)
        self.b_cpu = _randn_bf16((N, K), 4, 1.0)
        self.a, self.b = self.a_cpu.to(dev), self.b_cpu.to(dev)
        self._impl = gemm_fp8_impl
        self.aq, self.as_inv = quant_fp8_blockwise_impl(self.a, turbo.float8_e4m3, -1, 128)
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
        rel = OG.max_rel_err(ref_t, out[rows])
        cos = OG.cosine(out[rows], ref_t)
        ok = bool(same and rel <= 1e-2 and cos >= 0.9999)
        return ok, f"quantized bytes bit-exact; 128 output rows vs oracle: max_rel_err={rel:.2e}, cosine={cos:.6f}"

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


def register(workloads):
    workloads["gemm_fp8_rowwise"] = GemmFp8Rowwise
    workloads["gemm_fp8_blockwise"] = GemmFp8Blockwise
    workloads["gemm_fp8_blockwise_k7168"] = lambda dev: GemmFp8Blockwise(dev, 16384, 4096, 7168)
    workloads["gemm_fp8_blockwise_8192"] = lambda dev: GemmFp8Blockwise(dev, 8192, 8192, 8192)
