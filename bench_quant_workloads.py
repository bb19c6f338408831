"""Quantizer workloads of bench.py: one per quantizer family of the hot path, at the operand shapes
of the GEMM configurations they feed.

A step quantizes (and, where the reference has the inverse op, de-quantizes) one tensor that is
resident in HBM; ``value`` is algorithmic bytes per second: every input element read once, every
output element written once, scales included. ``dominant()`` is the quantizer kernel alone. Every
workload checks the bytes and scales of a slice against the CPU oracle, bit for bit, and times the
reference's CPU formulas (torch for FP8, the numpy oracle for MX) on a bounded slice.
"""

from __future__ import annotations

import os
import time

import numpy as np
import torch

HBM_PEAK_GBS = 8000.0


def _randn_bf16(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)


def _u8(t):
    return t.contiguous().view(torch.uint8).cpu().numpy()


def _f32(t):
    return t.float().cpu().numpy()


class _QuantBase:
    unit = "GB/s"
    bound = "hbm"
    dtype = "f32"
    metric = "quantize GB/s (algorithmic bytes) & fraction of HBM peak"
    graph_dominant = True  # kernels of tens of microseconds: time replays of a captured batch

    def rotate(self):
        """Point ``self.x`` at the next of several identical copies of the input (at least 640 MiB
        together): a kernel timed over the rotation reads from HBM; one that re-reads a single
        tensor of up to 256 MB is served by the Infinity Cache."""
        x = getattr(self, "x", None)
        if x is None:
            return
        if not hasattr(self, "_ring"):
            nbytes = x.numel() * x.element_size()
            n = max(2, min(24, -(-(640 << 20) // nbytes)))
            self._ring = [x] + [x.detach().clone().requires_grad_(x.requires_grad) for _ in range(n - 1)]
            self._pos = 0
        self._pos = (self._pos + 1) % len(self._ring)
        self.x = self._ring[self._pos]

    def _cpu(self, fn, nbytes, what):
        fn()
        times = []
        t_end = time.perf_counter() + 10.0
        while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 20):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        med = sorted(times)[len(times) // 2]
        return dict(value=round(nbytes / med / 1e9, 3), unit="GB/s", cores=torch.get_num_threads(), kind="port",
                    sample=f"{what}, median of {len(times)} runs, {os.cpu_count()} logical CPUs visible")


class HbmStream(_QuantBase):
    """The yardstick of the HBM-bound kernels: what plain streaming kernels of the same traffic shape
    reach on this GPU, measured by the same harness (rotating inputs, graph replays). The dominant
    kernel reads a 16384 x 7168 bf16 tensor and writes one fp8-sized byte per element (the traffic
    ratio of a quantizer, 3 bytes per element) with torch's elementwise cast; the other entries are a
    same-size copy (2 + 2 bytes per element), a fill (writes only) and a reduction (reads only)."""

    name = "hbm_streaming_yardstick_16384x7168_bf16 (torch elementwise cast to fp8, copy)"
    metric = "plain streaming GB/s & fraction of HBM peak"
    dominant_name = "torch elementwise bf16 -> float8_e4m3fn cast (reads 2 B, writes 1 B per element)"
    dtype = "bf16 (byte movement)"

    def __init__(self, dev, M=16384, N=7168):
        self.M, self.N = M, N
        self.x_cpu = _randn_bf16((M, N), 5, 1.0)
        self.x = self.x_cpu.to(dev)
        self.q = torch.empty((M, N), dtype=torch.float8_e4m3fn, device=dev)
        self.y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
        self.big = torch.empty((4 * M, N), dtype=torch.bfloat16, device=dev)

    def dominant_work(self):
        return 3.0 * self.M * self.N

    step_work = dominant_work

    def dominant(self):
        self.q.copy_(self.x)
        return self.q

    step = dominant

    def _copy(self):
        self.y.copy_(self.x)
        return self.y

    def _fill(self):
        self.y.zero_()
        return self.y

    def _fill_big(self):
        self.big.zero_()
        return self.big

    def _read(self):
        return self.x.view(torch.int32).amax()

    def kernels(self):
        # a pure write stream and a pure read stream beside the copy: what the two directions of
        # the memory system give on their own (a quantizer that emits two outputs, a gather that
        # writes eight rows per row read, are write-heavy)
        n = float(self.M * self.N)
        # (the 235 MB fill fits the 256 MB Infinity Cache, which absorbs repeated writes of the same
        # lines; the fill of four times that size has to reach HBM)
        return [("copy_bf16_to_bf16", self._copy, 4.0 * n), ("fill_write_only", self._fill, 2.0 * n),
                ("fill_write_only_940MB", self._fill_big, 8.0 * n), ("amax_read_only", self._read, 2.0 * n)]

    def check(self):
        ok = torch.equal(self._copy(), self.x) and torch.equal(self.dominant().float(), self.x.to(torch.float8_e4m3fn).float())
        return bool(ok), "copy returns the input; cast equals torch's own cast (library kernels: nothing of this build is checked here)"

    def cpu_baseline(self):
        x = self.x_cpu[:2048]
        y = torch.empty_like(x)
        return self._cpu(lambda: y.copy_(x), 4.0 * x.numel(), "torch CPU copy of 2048 rows")


class QuantRowwise(_QuantBase):
    """Rowwise FP8 quantize (last axis) + dequantize of an 8192 x 8192 bf16 GEMM operand."""

    name = "fp8_e4m3_rowwise_quant_dequant_8192x8192_bf16 (axis -1)"
    dominant_name = "quant_rowwise_inner_kernel (row parked in registers between amax and cast)"

    def __init__(self, dev, M=8192, N=8192):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.core.low_precision import ScalingGranularity as G

        self.turbo, self.G, self.M, self.N = turbo, G, M, N
        self.x_cpu = _randn_bf16((M, N), 11, 0.02)
        self.x = self.x_cpu.to(dev)

    def step_work(self):
        return 6.0 * self.M * self.N + 8.0 * self.M

    def dominant_work(self):
        return 3.0 * self.M * self.N + 4.0 * self.M

    def dominant(self):
        return self.turbo.ops.quantize_fp8(self.x, self.turbo.float8_e4m3, self.G.ROWWISE, axis=-1)

    def step(self):
        q, s = self.dominant()
        return self.turbo.ops.dequantize_fp8(q, torch.bfloat16, self.G.ROWWISE, axis=-1, scale_inv=s)

    def check(self):
        from oracle import quantize as Q

        q, s = self.dominant()
        y = self.turbo.ops.dequantize_fp8(q, torch.bfloat16, self.G.ROWWISE, axis=-1, scale_inv=s)
        rows = np.r_[0:128, self.M - 128 : self.M]
        oq, os_ = Q.fp8_rowwise(self.x_cpu.float().numpy()[rows], -1, "e4m3")
        same = np.array_equal(_u8(q)[rows], oq) and np.array_equal(_f32(s)[rows].view(np.int32), os_.view(np.int32))
        oy = torch.from_numpy(Q.fp8_dequant(oq, os_, "e4m3")).to(torch.bfloat16)
        same = same and torch.equal(y.cpu()[rows], oy)
        return bool(same), "256 rows: bytes, scale_inv and de-quantized bf16 bit-exact vs oracle"

    def cpu_baseline(self):
        from oracle import cpu_reference as R

        def fn():
            q, _, sinv = R.quantize_fp8_rowwise_ref(self.x_cpu, torch.float8_e4m3fn, axis=-1)
            R.dequantize_fp8_ref(q, torch.bfloat16, sinv)

        return self._cpu(fn, self.step_work(), "full 8192x8192 quantize + dequantize")


class QuantBlockwise(_QuantBase):
    """1x128 (and 128x1) blockwise FP8 quantize of a [16384, 7168] activation."""

    def __init__(self, dev, dual=False, M=16384, N=7168):
        from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

        self.qi, self.dual, self.M, self.N = qi, dual, M, N
        self.name = f"fp8_e4m3_blockwise_{'1x128+128x1_dual' if dual else '1x128'}_quant_{M}x{N}_bf16"
        self.dominant_name = ("quant_block128_kernel (one 128x128 tile per workgroup, row and column blocks)" if dual else
                              "quant_rows128_kernel (stream without LDS: 16 lanes per 1x128 block, four blocks of four rows per wavefront)")
        self.x_cpu = _randn_bf16((M, N), 12)
        self.x = self.x_cpu.to(dev)

    def step_work(self):
        n = self.M * self.N
        return (4.0 if self.dual else 3.0) * n + 4.0 * n / 128 * (2 if self.dual else 1)

    dominant_work = step_work

    def dominant(self):
        if self.dual:
            return self.qi.quant_fp8_blockwise_dual_impl(self.x, torch.float8_e4m3fn, 128)
        return self.qi.quant_fp8_blockwise_impl(self.x, torch.float8_e4m3fn, -1, 128)

    step = dominant

    def check(self):
        from oracle import quantize as Q

        out = self.dominant()
        x = self.x_cpu.float().numpy()[:256]
        oq, os_ = Q.fp8_blockwise(x, 1, "e4m3", 128)
        same = np.array_equal(_u8(out[0])[:256], oq) and np.array_equal(_f32(out[1])[:256].view(np.int32), os_.view(np.int32))
        if self.dual:
            cq, cs = Q.fp8_blockwise(x, 0, "e4m3", 128)
            same = same and np.array_equal(_u8(out[2])[:256], cq) and np.array_equal(_f32(out[3])[:2].view(np.int32), cs.view(np.int32))
        return bool(same), "first 256 rows: bytes and scale_inv bit-exact vs oracle"

    def cpu_baseline(self):
        from oracle import cpu_reference as R

        rows = 4096
        x = self.x_cpu[:rows]

        def fn():
            R.quantize_fp8_blockwise_ref(x, torch.float8_e4m3fn, 1, 128)
            if self.dual:
                R.quantize_fp8_blockwise_ref(x, torch.float8_e4m3fn, 128, 1)

        return self._cpu(fn, self.step_work() * rows / self.M, f"first {rows} rows")


class QuantBlockwiseWeight(_QuantBase):
    """128x128-tile FP8 quantize of the expert weights [32, 4096, 7168]."""

    name = "fp8_e4m3_blockwise_128x128_weight_quant_32x4096x7168_bf16"
    dominant_name = "quant_block128_kernel (one 128x128 tile per workgroup, tile scale)"
    graph_dominant = False

    def __init__(self, dev, B=32, M=4096, N=7168):
        from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

        self.qi, self.B, self.M, self.N = qi, B, M, N
        self.w_cpu = _randn_bf16((B, M, N), 13)
        self.w = self.w_cpu.to(dev)

    def step_work(self):
        n = self.B * self.M * self.N
        return 3.0 * n + 4.0 * n / (128 * 128)

    dominant_work = step_work

    def dominant(self):
        return self.qi.quant_fp8_blockwise_for_weight_impl(self.w, torch.float8_e4m3fn, 128)

    step = dominant

    def check(self):
        from oracle import quantize as Q

        q, s = self.dominant()
        same = True
        for b in (0, self.B - 1):
            oq, os_ = Q.fp8_blockwise_weight(self.w_cpu[b].float().numpy(), "e4m3", 128)
            same = same and np.array_equal(_u8(q[b]), oq) and np.array_equal(_f32(s[b]).view(np.int32), os_.view(np.int32))
        return bool(same), "experts 0 and 31: bytes and scale_inv bit-exact vs oracle"

    def cpu_baseline(self):
        from oracle import cpu_reference as R

        w = self.w_cpu[0]
        return self._cpu(lambda: R.quantize_fp8_blockwise_ref(w, torch.float8_e4m3fn, 128, 128), self.step_work() / self.B,
                         "one expert's weight of 32")


class QuantGrouped(_QuantBase):
    """Fused grouped row + column blockwise quantize of the routed tokens [32768, 7168], 32 experts."""

    name = "fp8_e4m3_grouped_row+col_blockwise_quant_32768x7168_bf16_32experts_zipf1.2"
    dominant_name = "quant_block128_occ4_kernel (grouped: row blocks + segment-padded column blocks from one read)"
    graph_dominant = False

    def __init__(self, dev, M=32768, N=7168, groups=32):
        from bench_workloads import _zipf_group_lens
        from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

        self.qi, self.M, self.N, self.groups = qi, M, N, groups
        self.lens = _zipf_group_lens(groups, M, 7)
        self.gl = torch.from_numpy(self.lens).to(dev)
        self.offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(self.gl)
        self.x_cpu = _randn_bf16((M, N), 14)
        self.x = self.x_cpu.to(dev)

    def step_work(self):
        n = self.M * self.N
        return 4.0 * n + 8.0 * n / 128

    dominant_work = step_work

    def dominant(self):
        return self.qi.quant_fp8_blockwise_segment_m_row_col_impl(self.x, torch.float8_e4m3fn, 128, self.gl, self.offs, 4096)

    step = dominant

    def check(self):
        """Experts that are small enough for the oracle to finish in seconds: all outputs of the
        whole call would need the full tensor, so the oracle runs on the rows of the first three
        non-empty experts re-based to a three-expert problem."""
        from oracle import quantize as Q

        qr, qc, sr, sc, plens, poffs = self.dominant()
        live = [g for g in range(self.groups) if self.lens[g] > 0][:3]
        offs = np.concatenate([[0], np.cumsum(self.lens)])
        poff = poffs.cpu().numpy()
        same = True
        for g in live:
            r0, r1 = int(offs[g]), int(offs[g + 1])
            x = self.x_cpu[r0:r1].float().numpy()
            o = Q.fp8_blockwise_segment_m_row_col(x, np.array([r1 - r0], dtype=np.int64), "e4m3", 128)
            rows_p = o["written_rows"]
            oqr, oqc, osr, osc = o["row"], o["col"][:rows_p], o["row_scale"], o["col_scale"][: rows_p // 128]
            p0 = int(poff[g])
            same = same and np.array_equal(_u8(qr[r0:r1]), oqr)
            same = same and np.array_equal(_f32(sr[:, r0:r1]).view(np.int32), osr.view(np.int32))
            same = same and np.array_equal(_u8(qc[p0 : p0 + rows_p]), oqc)
            same = same and np.array_equal(_f32(sc[p0 // 128 : (p0 + rows_p) // 128]).view(np.int32), osc.view(np.int32))
        return bool(same), f"experts {live}: row / column bytes and scales bit-exact vs oracle"

    def cpu_baseline(self):
        from oracle import cpu_reference as R

        rows = 4096
        x = self.x_cpu[:rows]

        def fn():
            R.quantize_fp8_blockwise_ref(x, torch.float8_e4m3fn, 1, 128)
            R.quantize_fp8_blockwise_ref(x, torch.float8_e4m3fn, 128, 1)

        return self._cpu(fn, self.step_work() * rows / self.M, f"row and column blocks of the first {rows} rows")


class QuantMx(_QuantBase):
    """MXFP8 / MXFP4 quantize (1x32 blocks, optionally also the transposed column direction) of a
    16384 x 16384 bf16 operand, plus the de-quantizer of the row output."""

    graph_dominant = False

    def __init__(self, dev, fp4=False, dual=False, M=16384, N=16384):
        from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

        self.qi, self.fp4, self.dual, self.M, self.N = qi, fp4, dual, M, N
        kind = "mxfp4_e2m1" if fp4 else "mxfp8_e4m3"
        self.fmt = "e2m1" if fp4 else "e4m3"
        self.name = f"{kind}_{'row+col_dual' if dual else 'row'}_quant_{M}x{N}_bf16" + ("" if dual else " (+ dequantize)")
        self.dominant_name = ("mx_quant_kernel (128x128 tile through LDS, E8M0 exponent from the amax bits)" if dual else
                              "mx_quant_rows_kernel (stream without LDS: 8 elements per lane, block amax over four lanes)")
        self.qdt = torch.float4_e2m1fn_x2 if fp4 else torch.float8_e4m3fn
        self._q = qi.quantize_mxfp4_impl if fp4 else qi.quantize_mxfp8_impl
        self._dq = qi.dequantize_mxfp4_impl if fp4 else qi.dequantize_mxfp8_impl
        self.x_cpu = _randn_bf16((M, N), 15)
        self.x = self.x_cpu.to(dev)

    def _qbytes(self):
        code = 0.5 if self.fp4 else 1.0
        n = self.M * self.N
        return (2.0 + (2 if self.dual else 1) * (code + 1.0 / 32)) * n

    def dominant_work(self):
        return self._qbytes()

    def step_work(self):
        code = 0.5 if self.fp4 else 1.0
        return self._qbytes() + (0.0 if self.dual else (code + 1.0 / 32 + 2.0) * self.M * self.N)

    def dominant(self):
        if self.dual:
            return self._q(self.x, self.qdt, None, 32, with_trans=True)
        return self._q(self.x, self.qdt, 1, 32)

    def step(self):
        out = self.dominant()
        if self.dual:
            return out
        return self._dq(out[0], torch.bfloat16, 1, 32, out[1])

    def check(self):
        from oracle import quantize as Q

        out = self.dominant()
        x = self.x_cpu.float().numpy()[:128]
        oq, os_ = Q.mx_quant_rowwise(x, self.fmt)
        same = np.array_equal(_u8(out[0])[:128], oq) and np.array_equal(_u8(out[1])[:128], os_)
        what = "first 128 rows: codes and E8M0 bytes bit-exact vs oracle"
        if self.dual:
            cq, cs = Q.mx_quant_colwise(x, self.fmt)
            cb = 64 if self.fp4 else 128  # code bytes of the first 128 rows in a transposed row
            same = same and np.array_equal(_u8(out[2])[:, :cb], cq[:, :cb]) and np.array_equal(_u8(out[3])[:, :4], cs[:, :4])
            what += " (row and transposed column outputs)"
        else:
            y = self._dq(out[0], torch.bfloat16, 1, 32, out[1])
            oy = torch.from_numpy(Q.mx_dequant(oq, os_, self.fmt)[:, : self.N].astype(np.float32)).to(torch.bfloat16)
            same = same and torch.equal(y.cpu()[:128], oy)
            what += "; de-quantized bf16 bit-exact"
        return bool(same), what

    def cpu_baseline(self):
        from oracle import quantize as Q

        rows = 512
        x = self.x_cpu[:rows].float().numpy()

        def fn():
            q, s = Q.mx_quant_rowwise(x, self.fmt)
            if self.dual:
                Q.mx_quant_colwise(x, self.fmt)
            else:
                Q.mx_dequant(q, s, self.fmt)

        return self._cpu(fn, self.step_work() * rows / self.M, f"numpy oracle on the first {rows} rows")


class SwigluWithProbs(_QuantBase):
    """SwiGLU with router probabilities between the two grouped GEMMs of the MoE configuration:
    32768 routed tokens, fc1 output 2 x 2048 -> 2048, forward + backward."""

    name = "swiglu_with_probs_32768tokens_hidden2048_bf16 (forward + backward)"
    metric = "gated activation GB/s (algorithmic bytes) & fraction of HBM peak"
    dominant_name = "glu_fwd_kernel<bf16, SiLU> (one workgroup per token row, 16-byte accesses)"
    dtype = "bf16 (fp32 arithmetic)"

    def __init__(self, dev, tokens=32768, hidden=2048):
        import primus_turbo.pytorch as turbo

        self.turbo, self.T, self.H = turbo, tokens, hidden
        self.x_cpu = _randn_bf16((tokens, 2 * hidden), 31, 1.0)
        g = torch.Generator().manual_seed(32)
        self.p_cpu = torch.rand(tokens, generator=g, dtype=torch.float32)
        self.x = self.x_cpu.to(dev).requires_grad_(True)
        self.p = self.p_cpu.to(dev).requires_grad_(True)
        self.go = _randn_bf16((tokens, hidden), 33, 1.0).to(dev)

    def dominant_work(self):  # 2 H read + H written per token, 2 bytes each, + the probability
        return 6.0 * self.T * self.H + 4.0 * self.T

    def step_work(self):  # backward: 3 H read, 2 H written
        return 16.0 * self.T * self.H + 12.0 * self.T

    def dominant(self):
        with torch.no_grad():
            return self.turbo.ops.swiglu_with_probs(self.x, self.p)

    def step(self):
        self.x.grad = None
        self.p.grad = None
        y = self.turbo.ops.swiglu_with_probs(self.x, self.p)
        y.backward(self.go)
        return y

    def check(self):
        from oracle import activation as A

        y = self.dominant().float().cpu().numpy()[:256]
        ref = A.glu_with_probs(self.x_cpu[:256].float().numpy(), self.p_cpu[:256].numpy(), "silu")
        ok = bool(np.all(np.abs(y - ref) <= 1.01 * 2.0 ** -8 * np.abs(ref) + 1e-6 * np.abs(ref).max()))
        return ok, "256 rows within one bf16 rounding of the float64 formula"

    def cpu_baseline(self):
        def fn():
            a, b = self.x_cpu[:4096].float().chunk(2, dim=-1)
            (torch.nn.functional.silu(a) * b * self.p_cpu[:4096, None]).to(torch.bfloat16)

        return self._cpu(fn, self.dominant_work() * 4096 / self.T, "forward of the first 4096 tokens in PyTorch")


class GluQuantGrouped(_QuantBase):
    """The step between the two grouped GEMMs of the MoE configuration in its fused form: fc1's
    output [32768, 2 x 2048] bf16 is read once by the grouped blockwise quantizer, which applies
    SwiGLU with the router probabilities on load and writes fc2's row codes, transposed
    segment-padded column codes and both scale tensors. The step also times the two-step form
    (activation kernel, then quantizer) whose extra 32768 x 2048 x 2 B write and re-read the fusion
    removes."""

    name = "swiglu_with_probs_fused_into_grouped_blockwise_quant_32768tokens_hidden2048_bf16"
    metric = "fused activation + quantize GB/s (algorithmic bytes) & fraction of HBM peak"
    dominant_name = "quant_block128_kernel<row + transposed column blocks, grouped, SiLU gate on load>"
    dtype = "bf16 in, e4m3 out (fp32 arithmetic)"

    def __init__(self, dev, tokens=32768, hidden=2048, groups=32):
        import primus_turbo.pytorch as turbo
        from primus_turbo.pytorch.kernels.quantization import quantization_impl as qi

        from bench_workloads import _zipf_group_lens

        self.turbo, self.qi, self.T, self.H = turbo, qi, tokens, hidden
        self.lens = _zipf_group_lens(groups, tokens, 7)
        self.gl = torch.from_numpy(self.lens).to(dev)
        self.offs = torch.ops.primus_turbo_cpp_extension.grouped_gemm_compute_offs(self.gl)
        self.x_cpu = _randn_bf16((tokens, 2 * hidden), 31, 1.0)
        g = torch.Generator().manual_seed(32)
        self.p_cpu = torch.rand(tokens, generator=g, dtype=torch.float32)
        self.x = self.x_cpu.to(dev)
        self.p = self.p_cpu.to(dev)

    def dominant_work(self):  # 2 H read (2 B each), H row codes + H column codes + scales written, + the probability
        n = self.T * self.H
        return 6.0 * n + 8.0 * n / 128 + 4.0 * self.T

    step_work = dominant_work

    def dominant(self):
        return self.qi.glu_quant_fp8_blockwise_segment_m_row_col_impl(self.x, self.p, None, "silu", torch.float8_e4m3fn, 128,
                                                                      self.gl, self.offs, True)

    step = dominant

    def two_step(self):
        y = self.turbo.ops.swiglu_with_probs(self.x, self.p)
        return self.qi.quant_fp8_blockwise_segment_m_row_col_t_impl(y, torch.float8_e4m3fn, 128, self.gl, self.offs)

    def kernels(self):
        n = self.T * self.H  # the two-step form moves 4 more bytes per element (bf16 activation out and in again)
        return [("two_step_swiglu_then_quantize", self.two_step, self.dominant_work() + 4.0 * n)]

    def check(self):
        a, b = self.dominant(), self.two_step()
        w = int(a[5][-1].item())
        same = (torch.equal(a[0].view(torch.uint8), b[0].view(torch.uint8)) and torch.equal(a[2], b[2])
                and torch.equal(a[1].view(torch.uint8)[:, :w], b[1].view(torch.uint8)[:, :w])
                and torch.equal(a[3][: w // 128], b[3][: w // 128]))
        from oracle import quantize as Q

        y = self.turbo.ops.swiglu_with_probs(self.x[:1024], self.p[:1024]).float().cpu().numpy()
        oq, os_ = Q.fp8_blockwise(y, 1, "e4m3", 128)
        same = same and np.array_equal(_u8(a[0])[:1024], oq)
        same = same and np.array_equal(_f32(a[2])[:, :1024].T.copy().view(np.int32), os_.view(np.int32))
        return bool(same), "codes and scales bit-identical with the two-step form; row codes of 1024 tokens bit-exact vs the oracle"

    def cpu_baseline(self):
        from oracle import cpu_reference as R

        rows = 2048

        def fn():
            a, b = self.x_cpu[:rows].float().chunk(2, dim=-1)
            y = (torch.nn.functional.silu(a) * b * self.p_cpu[:rows, None]).to(torch.bfloat16)
            R.quantize_fp8_blockwise_ref(y, torch.float8_e4m3fn, 1, 128)
            R.quantize_fp8_blockwise_ref(y, torch.float8_e4m3fn, 128, 1)

        return self._cpu(fn, self.dominant_work() * rows / self.T, f"first {rows} tokens: PyTorch SwiGLU, then row and column blockwise quantize")


class GluQuantGroupedMx(GluQuantGrouped):
    """The same step for the MXFP8 recipe: the grouped MX quantizer applies SwiGLU with the router
    probabilities on load and writes fc2's row codes (groups padded to 32 rows), transposed
    column codes (groups padded to 128) and both E8M0 scale arrays."""

    name = "swiglu_with_probs_fused_into_grouped_mxfp8_quant_32768tokens_hidden2048_bf16"
    dominant_name = "mx_quant_kernel<e4m3, row + transposed column blocks, grouped, SiLU gate on load>"
    dtype = "bf16 in, e4m3 + e8m0 out (fp32 arithmetic)"

    def dominant_work(self):  # 2 H read (2 B each), H row codes + H column codes + a scale byte per 32 each, + the probability
        n = self.T * self.H
        return 6.0 * n + 2.0 * n / 32 + 4.0 * self.T

    step_work = dominant_work

    def dominant(self):
        return self.qi.glu_grouped_quantize_mx_impl(self.x, self.p, None, "silu", torch.float8_e4m3fn, self.gl, self.offs, True)

    step = dominant

    def two_step(self):
        y = self.turbo.ops.swiglu_with_probs(self.x, self.p)
        return self.qi.grouped_quantize_mxfp8_impl(y, torch.float8_e4m3fn, None, 32, self.gl, self.offs, with_trans=True)

    def check(self):
        a, b = self.dominant(), self.two_step()
        mr, mc = int(a[5][-1].item()), int(a[7][-1].item())
        u8 = lambda t: t.view(torch.uint8)  # noqa: E731
        same = (torch.equal(u8(a[0])[:mr], u8(b[0])[:mr]) and torch.equal(u8(a[1])[:mr], u8(b[1])[:mr])
                and torch.equal(u8(a[2])[:, :mc], u8(b[2])[:, :mc]) and torch.equal(u8(a[3])[:, : mc // 32], u8(b[3])[:, : mc // 32]))
        from oracle import quantize as Q

        rows = int(self.lens[0])  # group 0 sits at the start of both layouts
        if rows > 0:
            y = self.turbo.ops.swiglu_with_probs(self.x[:rows], self.p[:rows]).float().cpu().numpy()
            oq, os_ = Q.mx_quant_rowwise(y, "e4m3")
            same = same and np.array_equal(_u8(a[0])[:rows], oq) and np.array_equal(_u8(a[1])[:rows], os_)
        return bool(same), f"codes and scales bit-identical with the two-step form; row codes of group 0 ({rows} tokens) bit-exact vs the oracle"

    def cpu_baseline(self):
        from oracle import quantize as Q

        rows = 512

        def fn():
            a, b = self.x_cpu[:rows].float().chunk(2, dim=-1)
            y = (torch.nn.functional.silu(a) * b * self.p_cpu[:rows, None]).to(torch.bfloat16).float().numpy()
            Q.mx_quant_rowwise(y, "e4m3")
            Q.mx_quant_colwise(y, "e4m3")

        return self._cpu(fn, self.dominant_work() * rows / self.T, f"first {rows} tokens: PyTorch SwiGLU, then the numpy MX oracle in both directions")


class MoePermute(_QuantBase):
    """MoE permute + unpermute around the expert bank of the MoE configuration: 4096 tokens with
    top-8 routing over 32 local experts (32768 routed rows), hidden 7168, bf16, rows padded per
    expert to 128. Dominant kernel: the permute copy (reads every token once, writes its 8 rows)."""

    name = "moe_permute_unpermute_4096tokens_top8_32experts_hidden7168_bf16 (pad 128)"
    metric = "MoE permute GB/s (algorithmic bytes) & fraction of HBM peak"
    dominant_name = "moe_permute_kernel (one workgroup per token row, 16-byte accesses, streaming stores)"
    dtype = "bf16 (byte copy; fp32 sum in unpermute)"

    def __init__(self, dev, tokens=4096, experts=32, topk=8, hidden=7168, pad=128):
        import primus_turbo.pytorch as turbo

        self.turbo, self.T, self.E, self.K, self.H, self.pad = turbo, tokens, experts, topk, hidden, pad
        rng = np.random.default_rng(41)
        self.topk_cpu = np.stack([rng.choice(experts, topk, replace=False) for _ in range(tokens)]).astype(np.int64)
        self.x_cpu = _randn_bf16((tokens, hidden), 42, 1.0)
        self.x = self.x_cpu.to(dev)
        self.topk = torch.from_numpy(self.topk_cpu).to(dev)
        self.ext = torch.ops.primus_turbo_cpp_extension
        pre = self.ext.permute_preprocessing(self.topk, experts, topk, pad, -1, 0)
        self.rmap, self.tpe, _, self.nd = pre
        self.rows = int(self.tpe.sum().item())
        self.out = torch.empty((self.rows, hidden), dtype=torch.bfloat16, device=dev)
        self.back = torch.empty((tokens, hidden), dtype=torch.bfloat16, device=dev)

    def dominant_work(self):  # every token read once, every permuted row (zero rows included) written once
        return 2.0 * self.H * (self.T + self.rows)

    def step_work(self):  # + the row map pass and the unpermute (reads the routed rows, writes the tokens)
        return 2.0 * self.dominant_work() + 8.0 * self.T * self.K

    def dominant(self):
        self.ext.permute(self.x, self.out, None, None, None, None, self.rmap, self.nd, self.pad, self.E, self.H, 0,
                         False, False, self.rows, 0)
        return self.out

    def step(self):
        pre = self.ext.permute_preprocessing(self.topk, self.E, self.K, self.pad, self.rows, 0)
        self.ext.permute(self.x, self.out, None, None, None, None, pre[0], pre[3], self.pad, self.E, self.H, 0, False,
                         False, self.rows, 0)
        self.ext.unpermute(self.out, self.back, None, None, pre[0], pre[3], self.E, self.H, False, 0)
        return self.back

    def check(self):
        from oracle import moe_permute as P

        rmap, tpe, _, _ = P.preprocess(self.topk_cpu, self.E, self.pad)
        ok = np.array_equal(self.rmap.cpu().numpy(), rmap) and np.array_equal(self.tpe.cpu().numpy(), tpe)
        want, _, _, written = P.permute(self.x_cpu.view(torch.int16).numpy(), rmap, self.E, self.rows, self.pad)
        ok = ok and bool(written.all()) and np.array_equal(self.dominant().view(torch.int16).cpu().numpy(), want)
        back = self.step()
        ok = ok and torch.equal(back.cpu(), (self.x_cpu.float() * self.K).to(torch.bfloat16))
        return bool(ok), "row map, tokens_per_expert and all permuted rows bit-exact vs oracle; unpermute = top-k x tokens"

    def cpu_baseline(self):
        from oracle import moe_permute as P

        x = self.x_cpu.view(torch.int16).numpy()
        rmap, _, _, _ = P.preprocess(self.topk_cpu, self.E, self.pad)

        def fn():
            P.permute(x, rmap, self.E, self.rows, self.pad)

        return self._cpu(fn, self.dominant_work(), "numpy oracle permute of the full workload (row map precomputed)")


def register(workloads):
    workloads["hbm_stream"] = HbmStream
    workloads["moe_permute"] = MoePermute
    workloads["swiglu_with_probs"] = SwigluWithProbs
    workloads["glu_quant_grouped"] = GluQuantGrouped
    workloads["glu_quant_grouped_mxfp8"] = GluQuantGroupedMx
    workloads["quant_rowwise"] = QuantRowwise
    workloads["quant_blockwise"] = lambda dev: QuantBlockwise(dev, False)
    workloads["quant_blockwise_dual"] = lambda dev: QuantBlockwise(dev, True)
    workloads["quant_blockwise_weight"] = QuantBlockwiseWeight
    workloads["quant_grouped"] = QuantGrouped
    workloads["quant_mxfp8"] = lambda dev: QuantMx(dev, False, False)
    workloads["quant_mxfp8_dual"] = lambda dev: QuantMx(dev, False, True)
    workloads["quant_mxfp4"] = lambda dev: QuantMx(dev, True, False)
    workloads["quant_mxfp4_dual"] = lambda dev: QuantMx(dev, True, True)
